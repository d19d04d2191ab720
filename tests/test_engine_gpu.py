"""The engine against the plain implementation, in float32 and in bfloat16: each request
alone and whole; with the last 32 tokens one by one; in batches of unequal lengths whose
shorter requests end earlier, one batch after another so that slots and pages are used
again; long decoding; the first tokens of a sequence; with and without HIP graphs."""
import functools
import random

import pytest
import torch

import plain_llama as pl
from conftest import TOL, rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
NAMES = ["A", "B", "C", "D", "E"]


def _requests(vocab, seed, lengths):
    rnd = random.Random(seed)
    return [[rnd.randrange(vocab) for _ in range(n)] for n in lengths]


@functools.lru_cache(maxsize=None)
def _plain_cached(folder, tokens, rounded):
    c, W = pl.read_config(folder), pl.read_weights(folder)
    return pl.forward(c, W, list(tokens), torch.bfloat16 if rounded else None)


def plain_logits(folder, tokens, dtype):
    return _plain_cached(folder, tuple(tokens), dtype == torch.bfloat16)


def make_engine(folder, dtype, max_tokens=1024, **kw):
    from bitnet_c_amd import Engine
    return Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, **kw)


LENGTHS = [1, 5, 33, 64, 65, 100, 150]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_requests_alone(model_folders, name, dtype):
    from bitnet_c_amd import StepEntry
    folder = model_folders(name, dtype)
    eng = make_engine(folder, dtype)
    for toks in _requests(eng.vocab_size, 11, LENGTHS):
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, toks, list(range(len(toks))))])
        eng.release(s)
        assert rel_err(got, plain_logits(folder, toks, dtype)) < TOL[dtype], len(toks)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_decode_steps_fold_their_norms_into_the_products(model_folders, name, graphs, monkeypatch):
    """bf16 decode steps of up to 16 rows: a part's last product adds itself to the stream and the next
    part's first product applies the norm, so that no norm kernel runs between them.  The logits agree
    with the plain implementation, and with the same steps run with every norm as a kernel of its own,
    within rounding."""
    from bitnet_c_amd import StepEntry, ops
    folder = model_folders(name, torch.bfloat16)
    reqs = _requests(pl.read_config(folder)["vocab"], 21, [70, 19, 33])
    n_dec = 12

    def run(fuse):
        monkeypatch.setattr(ops, "FUSE_NORMS", fuse)
        calls = {"into": 0, "pre": 0, "norm": 0}
        real = {n: getattr(ops, n) for n in ("linear_into_stream", "linear_prenorm", "linear_swiglu_prenorm", "add_rmsnorm")}
        monkeypatch.setattr(ops, "linear_into_stream", lambda *a, **k: (calls.__setitem__("into", calls["into"] + 1), real["linear_into_stream"](*a, **k))[1])
        monkeypatch.setattr(ops, "linear_prenorm", lambda *a, **k: (calls.__setitem__("pre", calls["pre"] + 1), real["linear_prenorm"](*a, **k))[1])
        monkeypatch.setattr(ops, "linear_swiglu_prenorm", lambda *a, **k: (calls.__setitem__("pre", calls["pre"] + 1), real["linear_swiglu_prenorm"](*a, **k))[1])
        monkeypatch.setattr(ops, "add_rmsnorm", lambda *a, **k: (calls.__setitem__("norm", calls["norm"] + 1), real["add_rmsnorm"](*a, **k))[1])
        eng = make_engine(folder, torch.bfloat16, use_graphs=graphs)
        slots = [eng.new_sequence() for _ in reqs]
        eng.step([StepEntry(s, r[:-n_dec], []) for s, r in zip(slots, reqs)])
        before = dict(calls)
        outs = []
        for t in range(n_dec):
            outs.append(eng.step([StepEntry(s, [r[len(r) - n_dec + t]], [0]) for s, r in zip(slots, reqs)]).clone())
        for s in slots:
            eng.release(s)
        for n in real:
            monkeypatch.setattr(ops, n, real[n])
        return torch.stack(outs, dim=1), {k: calls[k] - before[k] for k in calls}    # [request, step, vocab]

    fused, n_fused = run(True)
    plain_k, n_plain = run(False)
    cfg = pl.read_config(folder)
    L = cfg["layers"]
    assert n_plain["into"] == 0 and n_plain["pre"] == 0 and n_fused["into"] > 0
    # Counted on the eager run (a graph's first run launches every kernel again for its warm-up and capture) and
    # where the feed-forward's width is a multiple of 8 (configuration A's is not: its feed-forward asks for the
    # plain norm and computes its last product the plain way, only the attention's output product folds).
    assert n_fused["pre"] > 0 or cfg["ffn"] % 8
    if not graphs and cfg["ffn"] % 8 == 0:
        assert n_fused["into"] == 2 * L * n_dec - n_dec          # every product that ends a part but the last layer's
        assert n_fused["pre"] == 2 * L * n_dec - n_dec           # every product that begins a part but the first layer's
        assert n_fused["norm"] == 2 * n_dec                      # the first layer's norm and the final norm
        assert n_plain["norm"] == (2 * L + 1) * n_dec
    for i, r in enumerate(reqs):
        want = plain_logits(folder, r, torch.bfloat16)[len(r) - n_dec:]
        assert rel_err(fused[i], want) < TOL[torch.bfloat16]
        assert rel_err(plain_k[i], want) < TOL[torch.bfloat16]
        assert rel_err(fused[i], plain_k[i]) < TOL[torch.bfloat16]


@pytest.mark.parametrize("small_matrices", [False, True])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_streamed_copies_of_the_weights_change_no_result(model_folders, name, small_matrices, monkeypatch):
    """A bf16 engine with a second copy of every weight matrix in the order its decode kernels read it, and one
    without: prompts (whole, and one of 100 tokens after 50, whose feed-forward ends in partial sums), decode steps of
    3 sequences and of 20 (graphs of 4 and 32 rows) give the plain implementation's logits either way, and the copies
    are no part of what a step is counted to read.  With small_matrices the staged gate/up kernel takes these tiny
    matrices too (it is meant for matrices of at least six column tiles a CU), so that its path through the
    feed-forward runs here at 13 to 64 rows."""
    from bitnet_c_amd import StepEntry, ops
    if small_matrices:
        monkeypatch.setattr(ops, "STAGED_MIN_TILES_PER_CU", 0)
    folder = model_folders(name, torch.bfloat16)
    vocab = pl.read_config(folder)["vocab"]
    reqs = _requests(vocab, 77, [150] + [40 + j for j in range(19)])
    n_dec = 6
    outs = {}
    for streamed in (False, True):
        eng = make_engine(folder, torch.bfloat16, max_tokens=4096, streamed_weights=streamed)
        m = eng.model
        assert m.has_streamed == streamed and (m.head.streamed is not None) == streamed
        assert all((l.streamed is not None) == (streamed and l.stream_bytes() > 0) for l in m.linears()) and m.linears()
        assert m.streamed_bytes() >= m.weight_bytes() * 0.5           # every matrix once more (padded), norms aside
        outs[streamed, "bytes"] = m.weight_bytes()
        s = eng.new_sequence()
        eng.step([StepEntry(s, reqs[0][:50], [])])
        chunk = eng.step([StepEntry(s, reqs[0][50:], list(range(100)))])
        eng.release(s)
        assert rel_err(chunk, plain_logits(folder, reqs[0], torch.bfloat16)[50:]) < TOL[torch.bfloat16]
        for group in (reqs[:3], reqs):
            slots = [eng.new_sequence() for _ in group]
            eng.step([StepEntry(q, r[:-n_dec], []) for q, r in zip(slots, group)])
            got = torch.stack([eng.step([StepEntry(q, [r[len(r) - n_dec + t]], [0]) for q, r in zip(slots, group)])
                               for t in range(n_dec)], dim=1)          # [request, step, vocab]
            for q in slots:
                eng.release(q)
            for i, r in enumerate(group):
                assert rel_err(got[i], plain_logits(folder, r, torch.bfloat16)[len(r) - n_dec:]) < TOL[torch.bfloat16], (streamed, i)
            outs[streamed, len(group)] = got
        eng.cache.check()
        assert eng._graphs.keys() >= {4, 32}
    assert outs[False, "bytes"] == outs[True, "bytes"]
    for n in (3, len(reqs)):
        assert rel_err(outs[True, n], outs[False, n]) < TOL[torch.bfloat16]


@pytest.mark.parametrize("name", NAMES)
def test_whole_requests_without_the_library(model_folders, name, monkeypatch):
    """bf16 with the library's matrix product switched off: prompts of more than 64 tokens then go
    through this library's own matrix-core kernel (with the SwiGLU epilogue where the feed-forward
    keeps gate and up interleaved); batches of 17 to 64 rows through the streaming kernel."""
    from bitnet_c_amd import StepEntry, ops
    folder = model_folders(name, torch.bfloat16)
    monkeypatch.setattr(ops, "LIBRARY_PRODUCTS", False)
    called = []
    real = ops.gemm_mfma
    monkeypatch.setattr(ops, "gemm_mfma", lambda *a, **k: (called.append(1), real(*a, **k))[1])
    eng = make_engine(folder, torch.bfloat16)
    for toks in _requests(eng.vocab_size, 11, [33, 65, 150, 300]):
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, toks, list(range(len(toks))))])
        eng.release(s)
        assert rel_err(got, plain_logits(folder, toks, torch.bfloat16)) < TOL[torch.bfloat16], len(toks)
    assert called
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_last_32_tokens_one_by_one(model_folders, name, dtype, graphs):
    from bitnet_c_amd import StepEntry
    folder = model_folders(name, dtype)
    eng = make_engine(folder, dtype, use_graphs=graphs)
    for toks in _requests(eng.vocab_size, 12, [33, 70, 129, 160]):
        ref = plain_logits(folder, toks, dtype)
        s = eng.new_sequence()
        n0 = len(toks) - 32
        got = [eng.step([StepEntry(s, toks[:n0], list(range(n0)))])]
        for t in toks[n0:]:
            got.append(eng.step([StepEntry(s, [t], [0])]))
        eng.release(s)
        got = torch.cat(got)
        assert rel_err(got, ref) < TOL[dtype], len(toks)
        # the first wrong token, if any, names the place
        per_row = (got.cpu().double() - ref.double()).abs().max(dim=1).values / ref.double().pow(2).mean().sqrt()
        assert int((per_row > TOL[dtype]).sum()) == 0, per_row.argmax()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_with_slot_reuse(model_folders, name, dtype, graphs):
    """Three batches one after another in a cache that holds just one of them.  In a batch the
    prompts (unequal) run in one step, then every request goes on one token a step until its own
    end; ended requests give their slots back while the others go on."""
    from bitnet_c_amd import StepEntry
    folder = model_folders(name, dtype)
    eng = make_engine(folder, dtype, max_tokens=64 * 9, use_graphs=graphs)
    rnd = random.Random(13)
    batches = [[(5, 3), (70, 40), (17, 20), (1, 9)], [(64, 1), (3, 66), (128, 5)], [(30, 30), (2, 2), (63, 2), (65, 10), (9, 31)]]
    for bi, batch in enumerate(batches):
        reqs = [[rnd.randrange(eng.vocab_size) for _ in range(p + d)] for p, d in batch]
        slots = [eng.new_sequence() for _ in batch]
        got = [[] for _ in batch]
        out = eng.step([StepEntry(slots[i], reqs[i][:p], list(range(p))) for i, (p, d) in enumerate(batch)])
        o = 0
        for i, (p, d) in enumerate(batch):
            got[i].append(out[o:o + p])
            o += p
        fed = [p for p, d in batch]
        live = list(range(len(batch)))
        while live:
            out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1])
                fed[i] += 1
            for i in [i for i in live if fed[i] == len(reqs[i])]:
                eng.release(slots[i])
            live = [i for i in live if fed[i] < len(reqs[i])]
        eng.cache.check()
        assert not eng.cache.live_slots()
        for i, toks in enumerate(reqs):
            assert rel_err(torch.cat(got[i]), plain_logits(folder, toks, dtype)) < TOL[dtype], (bi, i)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_batch_and_cut_do_not_change_logits_beyond_rounding(model_folders, name, dtype):
    """The same request alone, in a batch with partners, cut into uneven pieces, and with its last 32
    tokens one by one (with and without graphs): float32 logits are equal bit for bit, because every
    kernel of that path sums a query's terms in one order however the step was cut; bfloat16 logits
    agree within rounding."""
    from bitnet_c_amd import StepEntry
    folder = model_folders(name, dtype)
    eng = make_engine(folder, dtype, max_tokens=2048)
    toks, p1, p2 = _requests(eng.vocab_size, 14, [90, 31, 140])
    s = eng.new_sequence()
    alone = eng.step([StepEntry(s, toks, list(range(90)))])
    eng.release(s)
    a, b, c = eng.new_sequence(), eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(a, p1, []), StepEntry(b, toks, list(range(90))), StepEntry(c, p2, [139])])
    batched = out[:90]
    for x in (a, b, c):
        eng.release(x)
    s = eng.new_sequence()
    pieces = [eng.step([StepEntry(s, toks[i:j], list(range(j - i)))]) for i, j in ((0, 1), (1, 64), (64, 65), (65, 90))]
    eng.release(s)
    one_by_one = []
    for graphs in (True, False):
        e2 = make_engine(folder, dtype, max_tokens=2048, use_graphs=graphs)
        s = e2.new_sequence()
        got = [e2.step([StepEntry(s, toks[:58], list(range(58)))])]
        got += [e2.step([StepEntry(s, [t], [0])]) for t in toks[58:]]
        e2.release(s)
        one_by_one.append(torch.cat(got))
    for other in (batched, torch.cat(pieces), *one_by_one):
        if dtype == torch.float32:
            assert torch.equal(other, alone)
        else:
            assert rel_err(other, alone) < 2e-2


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(model_folders, dtype):
    """300 tokens decoded one by one after a short prompt, across several pages and split
    plans, in a batch whose partner is much shorter."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("A", dtype)
    eng = make_engine(folder, dtype, max_tokens=1024)
    long_req, short_req = _requests(eng.vocab_size, 15, [310, 12])
    a, b = eng.new_sequence(), eng.new_sequence()
    got = [eng.step([StepEntry(a, long_req[:10], list(range(10))), StepEntry(b, short_req[:2], [])])[:10]]
    for i in range(10, 310):
        ent = [StepEntry(a, [long_req[i]], [0])]
        j = i - 10 + 2
        if j < len(short_req):
            ent.append(StepEntry(b, [short_req[j]], []))
        elif j == len(short_req):
            eng.release(b)
        got.append(eng.step(ent)[:1])
    eng.release(a)
    assert rel_err(torch.cat(got), plain_logits(folder, long_req, dtype)) < TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens_of_a_sequence(model_folders, dtype):
    """A sequence that starts with one token and grows by one: positions 0, 1, 2 are the places
    where an off-by-one in lengths or in the first page shows."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("B", dtype)
    eng = make_engine(folder, dtype)
    toks = _requests(eng.vocab_size, 16, [6])[0]
    s = eng.new_sequence()
    got = torch.cat([eng.step([StepEntry(s, [t], [0])]) for t in toks])
    eng.release(s)
    ref = plain_logits(folder, toks, dtype)
    for i in range(6):
        assert rel_err(got[i:i + 1], ref[i:i + 1]) < TOL[dtype], i


def test_errors_change_nothing(model_folders):
    from bitnet_c_amd import StepEntry
    from bitnet_c_amd.engine import StepError
    folder = model_folders("A", torch.float32)
    eng = make_engine(folder, torch.float32, max_tokens=128)
    s = eng.new_sequence()
    ref = eng.step([StepEntry(s, [1, 2, 3], [2])])
    for bad in ([StepEntry(s, [256], [0])], [StepEntry(s, [-1], [0])], [StepEntry(s, [], [])],
                [StepEntry(s, [1], [1])], [StepEntry(s, [1] * 200, [])], [StepEntry(99, [1], [0])],
                [StepEntry(s, [1], [0]), StepEntry(s, [2], [0])], []):
        with pytest.raises(StepError):
            eng.step(bad)
        assert eng.length(s) == 3
    eng.release(s)
    s2 = eng.new_sequence()
    again = eng.step([StepEntry(s2, [1, 2, 3], [2])])
    assert torch.equal(again, ref)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_a_step_that_mixes_single_tokens_and_a_chunk_all_past_position_zero(model_folders, name, dtype):
    """One step with a sequence that goes on by one token, a sequence that goes on by a chunk of 37 tokens
    (across a page's edge), another single token, and a new sequence's whole prompt: every row of every one
    matches the plain implementation, and in float32 the bits of the same rows run alone."""
    from bitnet_c_amd import StepEntry
    folder = model_folders(name, dtype)
    eng = make_engine(folder, dtype, max_tokens=2048)
    r_one, r_chunk, r_two, r_new = _requests(eng.vocab_size, 41, [72, 100, 6, 20])
    a, b, c, d = (eng.new_sequence() for _ in range(4))
    eng.step([StepEntry(a, r_one[:71], []), StepEntry(b, r_chunk[:40], []), StepEntry(c, r_two[:5], [])])
    out = eng.step([StepEntry(a, r_one[71:], [0]), StepEntry(b, r_chunk[40:77], list(range(37))),
                    StepEntry(c, r_two[5:], [0]), StepEntry(d, r_new, [19, 0])])
    assert out.shape[0] == 1 + 37 + 1 + 2
    want = [plain_logits(folder, r_one, dtype)[71:72], plain_logits(folder, r_chunk, dtype)[40:77],
            plain_logits(folder, r_two, dtype)[5:6], plain_logits(folder, r_new, dtype)[[19, 0]]]
    o = 0
    for w in want:
        assert rel_err(out[o:o + w.shape[0]], w) < TOL[dtype], o
        o += w.shape[0]
    # the chunk goes on: its later tokens see what the mixed step stored
    rest = eng.step([StepEntry(b, r_chunk[77:], list(range(23)))])
    assert rel_err(rest, plain_logits(folder, r_chunk, dtype)[77:]) < TOL[dtype]
    for x in (a, b, c, d):
        eng.release(x)
    if dtype == torch.float32:
        s = eng.new_sequence()
        eng.step([StepEntry(s, r_chunk[:40], [])])
        alone = eng.step([StepEntry(s, r_chunk[40:77], list(range(37)))])
        eng.release(s)
        assert torch.equal(alone, out[1:38])
    eng.cache.check()


def test_a_step_that_fails_halfway_leaves_nothing_behind(model_folders):
    """An error inside the forward pass (here: raised by a tap in the second layer) after the step's pages
    were taken: the pages go back, the lengths stay, and the same step runs afterwards as if nothing had been."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("A", torch.float32)
    eng = make_engine(folder, torch.float32, max_tokens=64 * 6)
    toks = _requests(eng.vocab_size, 43, [200])[0]
    s = eng.new_sequence()
    eng.step([StepEntry(s, toks[:60], [])])
    free = eng.cache.groups[0].pool.n_free

    def tap(point, entry, stream, ctx):
        if entry == 1:
            raise RuntimeError("boom")
    eng.tap = tap
    for n in (1, 100):                                       # a decode step and a chunk of two more pages
        with pytest.raises(RuntimeError):
            eng.step([StepEntry(s, toks[60:60 + n], [0])])
        assert eng.length(s) == 60 and eng.cache.groups[0].pool.n_free == free
        eng.cache.check()
    eng.tap = None
    got = torch.cat([eng.step([StepEntry(s, toks[60:160], list(range(100)))]), eng.step([StepEntry(s, [toks[160]], [0])])])
    assert rel_err(got, plain_logits(folder, toks[:161], torch.float32)[60:]) < TOL[torch.float32]
    eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_graphs_are_made_at_a_batch_s_start_and_never_between_tokens(model_folders, dtype):
    """prepare_decode(n) captures what decode steps of up to n sequences replay; afterwards sequences grow
    through page edges and through every power of two of pages, end one by one (the batch shrinks from five
    rows to one), and no further capture happens; the logits stay the plain ones all the way."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("C", dtype)                       # position limit 2,048
    eng = make_engine(folder, dtype, max_tokens=64 * 40, max_seq_len=1100)
    assert eng.max_pages == 18
    rnd = random.Random(44)
    ends = [1040, 80, 300, 20, 131]
    reqs = [[rnd.randrange(eng.vocab_size) for _ in range(n)] for n in ends]
    eng.prepare_decode(len(reqs))
    built = eng.graphs_built
    assert sorted(eng._graphs) == [1, 2, 4, 8] and built == 4          # five sequences: the step of eight rows and all below
    slots = [eng.new_sequence() for _ in reqs]
    fed = [10, 3, 60, 1, 64]
    eng.step([StepEntry(s, r[:f], []) for s, r, f in zip(slots, reqs, fed)])
    got = [[] for _ in reqs]
    live = list(range(len(reqs)))
    while live:
        out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
            fed[i] += 1
        for i in [i for i in live if fed[i] == ends[i]]:
            eng.release(slots[i])
        live = [i for i in live if fed[i] < ends[i]]
    assert eng.graphs_built == built
    for i, r in enumerate(reqs):
        n = len(got[i])
        assert rel_err(torch.cat(got[i]), plain_logits(folder, r, dtype)[-n:]) < TOL[dtype], i
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_through_the_engine(model_folders, dtype, tmp_path):
    """Weights made so that a fault shows: in a one-layer model whose q and k projections pick out
    one embedding dimension each and whose positions are not rotated there (the lowest frequency at
    a huge theta), token `mark` at a far position takes all the attention of the last token `probe`;
    without the marked token the logits differ by several times their size, and with it they match
    the plain implementation wherever it lies (first position, a page's edge, the decoded part)."""
    import json, os
    from bitnet_c_amd import StepEntry
    from bitnet_c_amd.config import LlamaConfig
    from bitnet_c_amd.weights import write_file, random_tensors
    from bitnet_c_amd.config import load_config
    cfg = dict(model_type="llama", vocab_size=50, hidden_size=32, intermediate_size=48, num_hidden_layers=1,
               num_attention_heads=2, num_key_value_heads=1, head_dim=16, max_position_embeddings=2048,
               rope_theta=1e12, rms_norm_eps=1e-5, tie_word_embeddings=False)
    c = LlamaConfig.from_dict(cfg)
    folder = str(tmp_path / "far")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(c.to_dict(), f)
    arch, _ = load_config(folder)
    t = random_tensors(arch.build_plan(c).expected_tensors(), 21, torch.float32)
    mark, probe = 7, 9
    E = t["model.embed_tokens.weight"]
    E[:, 0] = 0
    E[:, 1] = 0
    E[mark, 0] = 1.0            # the key of `mark` comes from embedding dimension 0,
    E[probe, 1] = 1.0           # the query of `probe` from dimension 1: the probe does not see itself
    # dimension 7 of a head is paired with 15 and turns at theta^(-14/16): no rotation over 1000 positions
    wq = torch.zeros_like(t["model.layers.0.self_attn.q_proj.weight"])
    wk = torch.zeros_like(t["model.layers.0.self_attn.k_proj.weight"])
    wq[7, 1] = wq[16 + 7, 1] = 60.0
    wk[7, 0] = 60.0
    t["model.layers.0.self_attn.q_proj.weight"], t["model.layers.0.self_attn.k_proj.weight"] = wq, wk
    t["model.layers.0.self_attn.v_proj.weight"] *= 20.0
    t["model.layers.0.self_attn.o_proj.weight"] *= 20.0
    if dtype == torch.bfloat16:
        t = {k: (v.to(torch.bfloat16) if v.dim() == 2 else v) for k, v in t.items()}
    write_file(os.path.join(folder, "model.safetensors"), t)
    eng = make_engine(folder, dtype, max_tokens=2048)
    rnd = random.Random(22)
    outs = {}
    for far in (0, 63, 64, 500, 958):
        toks = [rnd.choice([x for x in range(50) if x not in (mark, probe)]) for _ in range(960)]
        toks[far] = mark
        toks[959] = probe
        s = eng.new_sequence()
        eng.step([StepEntry(s, toks[:900], [])])
        for tk in toks[900:959]:
            eng.step([StepEntry(s, [tk], [])])
        got = eng.step([StepEntry(s, [probe], [0])])
        eng.release(s)
        ref = plain_logits(folder, toks, dtype)[959:960]
        assert rel_err(got, ref) < TOL[dtype], far
        outs[far] = got
        # and the marked key matters: without it the logits differ by far more than the tolerance
        toks2 = list(toks)
        toks2[far] = 3
        assert rel_err(plain_logits(folder, toks2, dtype)[959:960], ref) > 20 * TOL[dtype], far


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replays_of_a_wide_batch(model_folders, dtype):
    """24 sequences decode together: at this width the bf16 products are the library's, inside the
    replayed graph.  Every replay is checked: against the same steps run without graphs (equal
    bits are demanded: the same kernels run) and against the plain implementation, with eager
    prompt steps of other sequences and synchronisations between the replays."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("C", dtype)
    rnd = random.Random(17)
    engines = [make_engine(folder, dtype, max_tokens=64 * 40, use_graphs=g) for g in (True, False)]
    vocab = engines[0].vocab_size
    reqs = [[rnd.randrange(vocab) for _ in range(3 + i + 7)] for i in range(24)]
    extra = [[rnd.randrange(vocab) for _ in range(20)] for _ in range(7)]
    outs = []
    for eng in engines:
        slots = [eng.new_sequence() for _ in reqs]
        got = [[] for _ in reqs]
        out = eng.step([StepEntry(s, r[:-7], [len(r) - 8]) for s, r in zip(slots, reqs)])
        for i in range(24):
            got[i].append(out[i:i + 1])
        for k in range(7):
            other = eng.new_sequence()                              # eager work between the replays
            eng.step([StepEntry(other, extra[k], [19])])
            eng.release(other)
            torch.cuda.synchronize()
            out = eng.step([StepEntry(s, [r[len(r) - 7 + k]], [0]) for s, r in zip(slots, reqs)])
            for i in range(24):
                got[i].append(out[i:i + 1])
        outs.append([torch.cat(g) for g in got])
    for i, r in enumerate(reqs):
        assert torch.equal(outs[0][i], outs[1][i]), i
        ref = plain_logits(folder, r, dtype)[len(r) - 8:]
        assert rel_err(outs[0][i], ref) < TOL[dtype], i


@pytest.mark.parametrize("dtype", DTYPES)
def test_more_sequences_than_a_graph_takes_and_a_long_context(model_folders, dtype):
    """70 sequences decode in one step (more than the replayed graphs hold: the step runs eagerly),
    and one sequence grows past 1,100 positions token by token, through several block-table widths."""
    from bitnet_c_amd import StepEntry
    folder = model_folders("A", dtype)
    eng = make_engine(folder, dtype, max_tokens=64 * 110)
    rnd = random.Random(18)
    reqs = [[rnd.randrange(eng.vocab_size) for _ in range(2 + i % 5 + 3)] for i in range(70)]
    slots = [eng.new_sequence() for _ in reqs]
    eng.step([StepEntry(s, r[:-3], []) for s, r in zip(slots, reqs)])
    got = [[] for _ in reqs]
    for k in range(3):
        out = eng.step([StepEntry(s, [r[len(r) - 3 + k]], [0]) for s, r in zip(slots, reqs)])
        for i in range(70):
            got[i].append(out[i:i + 1])
    for i in (0, 1, 33, 68, 69):
        assert rel_err(torch.cat(got[i]), plain_logits(folder, reqs[i], dtype)[-3:]) < TOL[dtype], i
    for s in slots:
        eng.release(s)
    folder = model_folders("C", dtype)                 # its position limit is 2,048
    eng = make_engine(folder, dtype, max_tokens=64 * 20)
    long_req = [rnd.randrange(eng.vocab_size) for _ in range(1130)]
    s = eng.new_sequence()
    outs = [eng.step([StepEntry(s, long_req[:1000], [999])])]
    for t in long_req[1000:]:
        outs.append(eng.step([StepEntry(s, [t], [0])]))
    eng.release(s)
    assert rel_err(torch.cat(outs), plain_logits(folder, long_req, dtype)[999:]) < TOL[dtype]
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
def test_forty_sequences_of_unequal_lengths_with_eight_kv_heads(model_folders, graphs):
    """More attention workgroups than CUs in a decode step: the kernel then hands them out by
    sequence length (the step context carries the order).  Every sequence's logits are the plain
    ones; sequences end at different steps, so the order changes from step to step."""
    from bitnet_c_amd import StepEntry
    dtype = torch.bfloat16
    folder = model_folders("F", dtype)
    eng = make_engine(folder, dtype, max_tokens=64 * 100, use_graphs=graphs)
    rnd = random.Random(21)
    reqs = [[rnd.randrange(eng.vocab_size) for _ in range(rnd.randrange(3, 90) + 2 + i % 4)] for i in range(40)]
    n_dec = [2 + i % 4 for i in range(40)]
    slots = [eng.new_sequence() for _ in reqs]
    eng.step([StepEntry(s, r[:-d], []) for s, r, d in zip(slots, reqs, n_dec)])
    got = [[] for _ in reqs]
    fed = [len(r) - d for r, d in zip(reqs, n_dec)]
    live = list(range(40))
    while live:
        out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
            fed[i] += 1
        live = [i for i in live if fed[i] < len(reqs[i])]
    for i in range(40):
        assert rel_err(torch.cat(got[i]), plain_logits(folder, reqs[i], dtype)[-n_dec[i]:]) < TOL[dtype], i


def test_cuts_and_batches_agree_at_the_benchmark_layer_sizes():
    """Two layers of the Llama-3.1-8B shape (bfloat16, random weights made on the device): the
    kernels at their real sizes, where a prompt's products go to the library and a decoded token's
    to the streaming kernel.  The same request whole, with its last 32 tokens one by one, and inside a
    batch of unequal partners: a float32 engine on the same (bfloat16) weights gives equal bits all three
    ways and agrees with the plain implementation, run on the CPU at this width; the bfloat16 engine
    agrees with them within what rounding looks like at this width."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors
    raw = dict(model_type="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    tensors = random_tensors(plan.expected_tensors(), 3, torch.bfloat16, device="cuda:0")
    engines = {}
    for dtype in (torch.bfloat16, torch.float32):
        model = DecoderModel(plan, dtype, "cuda:0")
        model.load(tensors)
        engines[dtype] = bn.Engine(model, max_tokens=16384)
    rnd = random.Random(31)
    toks, p1, p2 = ([rnd.randrange(cfg.vocab_size) for _ in range(n)] for n in (300, 70, 513))
    last = list(range(268, 300))
    # the plain implementation at this width, on the CPU, in float32 on the same (bfloat16) weights: all 300
    # tokens through the two layers, the final norm and the output matrix for the last 32 only
    W = {k: v.float().cpu() for k, v in tensors.items()}
    del tensors
    c = dict(dim=cfg.hidden_size, ffn=cfg.intermediate_size, layers=2, heads=32, kv_heads=8, head_dim=128,
             vocab=cfg.vocab_size, theta=cfg.rope_theta, eps=cfg.rms_norm_eps, tied=False, rope_scaling=raw["rope_scaling"])
    x = W["model.embed_tokens.weight"][torch.tensor(toks)]
    inv = pl.rope_inv_freq(128, c["theta"], c["rope_scaling"])
    for l in range(2):
        x = pl.decoder_layer(x, torch.arange(300), W, l, c, inv)
    plain_ref = pl.linear(pl.rmsnorm(x[268:], W["model.norm.weight"], c["eps"]), W["lm_head.weight"])
    del W

    def run(eng):
        s = eng.new_sequence()
        whole = eng.step([bn.StepEntry(s, toks, last)])
        eng.release(s)
        s = eng.new_sequence()
        eng.step([bn.StepEntry(s, toks[:268], [])])
        one_by_one = torch.cat([eng.step([bn.StepEntry(s, [t], [0])]) for t in toks[268:]])
        eng.release(s)
        a, b, c = eng.new_sequence(), eng.new_sequence(), eng.new_sequence()
        out = eng.step([bn.StepEntry(a, p1, []), bn.StepEntry(b, toks[:268], []), bn.StepEntry(c, p2, [512])])
        rows = []
        for t in toks[268:]:                       # the partners go on too, with tokens of their own
            o = eng.step([bn.StepEntry(a, [5], []), bn.StepEntry(b, [t], [0]), bn.StepEntry(c, [7], [0])])
            rows.append(o[:1])
        for x in (a, b, c):
            eng.release(x)
        # the prompt in two steps, the second of 100 tokens: at 64 to 128 rows a feed-forward's last product is left
        # as partial sums over ranges of K (4,096 x 14,336 here) that the kernels of the next norm add up
        s = eng.new_sequence()
        eng.step([bn.StepEntry(s, toks[:200], [])])
        chunk = eng.step([bn.StepEntry(s, toks[200:], list(range(68, 100)))])
        eng.release(s)
        # twenty sequences that decode together, sequence j from the first 268 + j tokens: steps of 20 rows (a
        # captured step of 32 rows, whose products have more rows than one tile of the matrix cores); row j of
        # step k holds the logits at position 268 + j + k
        seqs = [eng.new_sequence() for _ in range(20)]
        eng.step([bn.StepEntry(q, toks[:268 + j], []) for j, q in enumerate(seqs)])
        wide = torch.cat([eng.step([bn.StepEntry(q, [toks[268 + j + k]], [0]) for j, q in enumerate(seqs)])
                          for k in range(12)])
        for q in seqs:
            eng.release(q)
        eng.cache.check()
        return whole, one_by_one, torch.cat(rows), chunk, wide

    wide_rows = torch.tensor([j + k for k in range(12) for j in range(20)], device="cuda:0")
    ref = run(engines[torch.float32])
    assert torch.equal(ref[1], ref[0]) and torch.equal(ref[2], ref[0])     # float32: no cut changes a bit
    assert torch.equal(ref[3], ref[0]) and torch.equal(ref[4], ref[0][wide_rows])
    assert rel_err(ref[0], plain_ref) < TOL[torch.float32]                 # and they are the plain implementation's
    got = run(engines[torch.bfloat16])
    assert engines[torch.bfloat16]._graphs.keys() >= {1, 4, 32}           # the decode steps were replayed from graphs
    # 32 x 128,256 logits: the largest of four million differences is no measure (rounding noise of
    # standard deviation s has its largest value near 5.5 s there).  What rounding looks like at this
    # width: a difference of about 1.4 % of the logits' root mean square, the same in every row, with
    # no value far outside it.  A fault (a wrong key, a lost column) breaks one of the three.
    rms = float(ref[0].double().pow(2).mean().sqrt())
    for i, g in enumerate(got):
        d = (g - (ref[0][wide_rows] if i == 4 else ref[0])).double()
        per_row = d.pow(2).mean(dim=1).sqrt() / rms
        assert float(per_row.max()) < 0.025, (i, per_row)
        assert float(per_row.max() / per_row.min()) < 2.0, (i, per_row)
        assert float(d.abs().max() / d.pow(2).mean().sqrt()) < 7.0, i


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_positions_beyond_the_original_context_with_the_8b_rotation_table(dtype):
    """A sequence of 8,260 tokens with the head size, theta and llama3 scaling of the Llama-3.1-8B shape
    (original context 8,192) at a narrow width: a prompt step that ends beyond position 8,192, then tokens one
    by one from there (the decode kernels work the rotation out of the position themselves), against the plain
    implementation.  With rotation in single precision an angle at position 8,200 is exact to about 5e-4, and
    a table or a position that is off by one shows far above the tolerance."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors
    raw = dict(model_type="llama", vocab_size=96, hidden_size=256, intermediate_size=344,
               num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
               max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    tensors = random_tensors(plan.expected_tensors(), 9, dtype, device="cuda:0")
    # queries and keys large enough that the rotation decides which keys a token attends to
    for name in ("model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.k_proj.weight"):
        tensors[name] = (tensors[name].float() * 12.0).to(dtype)
    model = DecoderModel(plan, dtype, "cuda:0")
    model.load(tensors)
    eng = bn.Engine(model, max_tokens=8320 + 64)
    T, fed = 8260, 8254
    rnd = random.Random(12)
    toks = [rnd.randrange(cfg.vocab_size) for _ in range(T)]
    W = {k: v.float().cpu() for k, v in tensors.items()}
    c = dict(dim=cfg.hidden_size, ffn=cfg.intermediate_size, layers=1, heads=2, kv_heads=1, head_dim=128,
             vocab=cfg.vocab_size, theta=cfg.rope_theta, eps=cfg.rms_norm_eps, tied=False, rope_scaling=raw["rope_scaling"])
    rt = None if dtype == torch.float32 else dtype
    inv = pl.rope_inv_freq(128, c["theta"], c["rope_scaling"])
    x = pl.decoder_layer(W["model.embed_tokens.weight"][torch.tensor(toks)], torch.arange(T), W, 0, c, inv, rt)
    want_rows = list(range(8190, 8196)) + list(range(fed - 4, T))          # around 8,192 and at the end
    xb = pl.rmsnorm(x[want_rows], W["model.norm.weight"], c["eps"])
    plain_ref = pl.linear(xb if rt is None else xb.to(rt).float(), W["lm_head.weight"])
    s = eng.new_sequence()
    got = [eng.step([bn.StepEntry(s, toks[:fed], [r for r in want_rows if r < fed])])]
    for t in toks[fed:]:
        got.append(eng.step([bn.StepEntry(s, [t], [0])]))
    got = torch.cat(got)
    assert rel_err(got, plain_ref) < TOL[dtype], rel_err(got, plain_ref)
    # the check can fail: with the last token one position too far the plain implementation gives other values
    tail = W["model.embed_tokens.weight"][torch.tensor(toks[8100:])]
    right = pl.decoder_layer(tail, torch.arange(8100, T), W, 0, c, inv, rt)
    one_off = pl.decoder_layer(tail, torch.cat([torch.arange(8100, T - 1), torch.tensor([T])]), W, 0, c, inv, rt)
    assert rel_err(one_off[-1:], right[-1:]) > 10 * TOL[dtype]
    eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("H,Hkv,lens", [(8, 8, [700]), (8, 8, [300, 9, 1500]), (40, 40, [520, 70])])
def test_decoding_with_the_split_plan_of_a_very_long_context(H, Hkv, lens, monkeypatch):
    """An engine whose sequences may grow to 131,072 tokens cuts the keys of a captured decode step for that length:
    up to 64 runs, of which a sequence of some hundred tokens fills the first few and leaves the rest empty, with heads
    of 128 that have a kv head each.  bfloat16 (float32 never splits its keys), against the plain implementation, with
    one key among the hundreds made to stand out so that a run that is lost or merged twice shows."""
    import bitnet_c_amd as bn
    from bitnet_c_amd import ops
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors
    if H * len(lens) <= 8:
        monkeypatch.setattr(ops, "DECODE_TARGET_WGS", 512)       # the most runs a launch can have (64), as a larger chip would ask for
    dtype = torch.bfloat16
    raw = dict(model_type="llama", vocab_size=96, hidden_size=64, intermediate_size=136, num_hidden_layers=2,
               num_attention_heads=H, num_key_value_heads=Hkv, head_dim=128, max_position_embeddings=131072,
               rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    tensors = random_tensors(plan.expected_tensors(), 19, dtype, device="cuda:0")
    for name in ("model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.k_proj.weight"):
        tensors[name] = (tensors[name].float() * 14.0).to(dtype)          # scores that tell keys apart
    model = DecoderModel(plan, dtype, "cuda:0")
    model.load(tensors)
    eng = bn.Engine(model, max_tokens=131072 + 4096)
    assert eng.max_seq_len == 131072
    n_splits, _ = ops.decode_splits(len(lens), H, Hkv, eng.max_seq_len, dtype)
    assert n_splits >= (64 if H * len(lens) <= 8 else 3)
    n_dec = 6
    reqs = _requests(96, 77, [n + n_dec for n in lens])
    W = {k: v.float().cpu() for k, v in tensors.items()}
    c = dict(dim=64, ffn=136, layers=2, heads=H, kv_heads=Hkv, head_dim=128, vocab=96, theta=cfg.rope_theta,
             eps=cfg.rms_norm_eps, tied=False, rope_scaling=None, act="silu")
    slots = [eng.new_sequence() for _ in reqs]
    eng.step([bn.StepEntry(s, r[:-n_dec], []) for s, r in zip(slots, reqs)])
    got = [[] for _ in reqs]
    for t in range(n_dec):
        lg = eng.step([bn.StepEntry(s, [r[len(r) - n_dec + t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(lg[i:i + 1].clone())
    assert eng._graphs, "the decode steps were meant to be replayed from a graph"
    for i, r in enumerate(reqs):
        want = pl.forward(c, W, r, dtype)[-n_dec:]
        assert rel_err(torch.cat(got[i]), want) < TOL[dtype], (i, len(r))
    for s in slots:
        eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_prompt_steps_are_replayed_from_graphs(model_folders, name, dtype, monkeypatch):
    """The first prompt step of a bucket (token rows, sequences, wanted places) runs eagerly, the second is recorded,
    later ones are replays with other sequences, other lengths inside the bucket, other places in the cache and other
    wanted rows: continuations of a prompt, mixed steps (a sequence with one token beside one with many), steps that
    want nothing.  float32: every step equals, bit for bit, the same step of an engine that never records prompt steps;
    bfloat16: within rounding (the padded step may pick another product kernel).  The graphs that an engine keeps are
    bounded: the one unused for longest goes."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.engine import step as step_mod
    monkeypatch.setattr(step_mod, "MAX_PROMPT_GRAPHS", 3)
    folder = model_folders(name, dtype)
    vocab = pl.read_config(folder)["vocab"]
    engines = [bn.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 64) for _ in range(2)]
    engines[1].prompt_graphs = False
    assert engines[0].prompt_graphs
    rnd = random.Random(5)
    toks = lambda n: [rnd.randrange(vocab) for _ in range(n)]
    # (new sequences' prompt lengths, continuation lengths of the sequences that live, single tokens for live sequences)
    script = [([40, 9], [], 0), ([33, 20], [], 0), ([50, 3], [], 0),           # bucket (64 rows, 2 seqs): eager, recorded, replayed
              ([], [30, 31], 0), ([], [17, 5], 2),                              # continuations; then mixed with two decoding rows
              ([100], [], 0), ([90], [], 0), ([70], [], 0),                    # (128, 1)
              ([3], [], 0), ([9], [], 0), ([16], [], 0),                        # (16, 1)
              ([20, 20, 20, 4], [], 0), ([10, 30, 1, 23], [], 0), ([5, 5, 5, 49], [], 0),   # (64, 4)
              ([44, 4], [], 0)]                                                  # (64, 2) again: its graph was dropped meanwhile
    outs = [[], []]
    for which, eng in enumerate(engines):
        rnd.seed(5)
        live = []
        for new, cont, singles in script:
            ent = []
            for n in new:
                s = eng.new_sequence()
                live.append(s)
                ent.append(bn.StepEntry(s, toks(n), [0, n - 1] if n > 1 else [0]))
            older = [s for s in live if s not in [e.slot for e in ent]]
            for n, s in zip(cont, older):
                ent.append(bn.StepEntry(s, toks(n), [n // 2]))
            for s in older[len(cont):len(cont) + singles]:
                ent.append(bn.StepEntry(s, toks(1), []))                      # a row that decodes, and wants nothing
            outs[which].append(eng.step(ent))
            if len(live) > 6:                                                  # slots are given back and used again
                for s in live[:4]:
                    eng.release(s)
                live = live[4:]
        eng.cache.check()
    eng = engines[0]
    assert eng.graphs_built >= 5 and len(eng._prompt_graphs) <= 3
    assert (64, 2, 4) in eng._prompt_seen and not engines[1]._prompt_graphs
    for i, (a, b) in enumerate(zip(*outs)):
        assert a.shape == b.shape
        if dtype == torch.float32:
            assert torch.equal(a, b), i
        else:
            assert rel_err(a, b) < TOL[dtype], i


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_graph_row_that_changes_its_owner_holds_nothing_of_the_former_one(model_folders, dtype):
    """A captured decode step keeps a block table at the engine's full width.  A long sequence decodes in row 0, ends, and a
    short one takes the row (and later no one does: the batch shrinks): the row's entries beyond the new owner's pages are
    zero, as the eager step's table has them, and a replayed step writes nothing but the new keys and values of the
    sequences it holds: every other place of the cache, the former owner's pages among them, keeps its bits."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.cache import PAGE
    folder = model_folders("A", dtype)
    eng = bn.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 16)
    vocab = eng.vocab_size
    long_, other, short = _requests(vocab, 55, [200, 70, 5])
    a, b = eng.new_sequence(), eng.new_sequence()
    eng.step([bn.StepEntry(a, long_, []), bn.StepEntry(b, other, [])])
    eng.step([bn.StepEntry(a, [1], [0]), bn.StepEntry(b, [2], [0])])           # a graph of two rows; row 0 holds a's four pages
    g = eng._graphs[2]
    assert int((g.tables_np[0, 0] != 0).sum()) >= 3
    eng.release(a)
    c = eng.new_sequence()
    eng.step([bn.StepEntry(c, short, [])])
    grp = eng.cache.groups[0]

    def step_and_diff(entries):
        k0, v0 = grp.k.clone(), grp.v.clone()
        out = eng.step(entries)
        torch.cuda.synchronize()
        changed = ((grp.k != k0) | (grp.k.isnan() != k0.isnan())).any(dim=0)      # [pages, Hkv, PAGE, hs] over the entries
        return out, {(int(p), int(o)) for p, _, o, _ in changed.nonzero().tolist()}, v0

    want = lambda slots: {(eng.cache.pages_of(0, s)[(eng.length(s) - 1) // PAGE], (eng.length(s) - 1) % PAGE) for s in slots}
    out, places, _ = step_and_diff([bn.StepEntry(c, [3], [0]), bn.StepEntry(b, [4], [0])])   # c in the row that a had
    assert places == want([c, b])
    assert len(eng.cache.pages_of(0, c)) == 1 and int((g.tables_np[0, 0, 1:] != 0).sum()) == 0
    # and the logits are those of the same sequences in an engine without graphs
    ref = bn.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 16, use_graphs=False)
    rc, rb = ref.new_sequence(), ref.new_sequence()
    ref.step([bn.StepEntry(rc, short, []), bn.StepEntry(rb, other + [2], [])])
    want_out = ref.step([bn.StepEntry(rc, [3], [0]), bn.StepEntry(rb, [4], [0])])
    assert torch.equal(out, want_out) if dtype == torch.float32 else rel_err(out, want_out) < TOL[dtype]
    # four sequences in a graph of four rows, then three: row 2 goes from a sequence of three pages to one of two, and
    # row 3 to nobody
    d, e = eng.new_sequence(), eng.new_sequence()
    eng.step([bn.StepEntry(d, other[:60] + long_[:70], []), bn.StepEntry(e, long_[:100], [])])
    eng.step([bn.StepEntry(s, [5 + i], [0]) for i, s in enumerate((c, b, d, e))])
    g4 = eng._graphs[4]
    assert int((g4.tables_np[0, 2] != 0).sum()) >= 2 and int((g4.tables_np[0, 3] != 0).sum()) >= 1
    eng.release(d)
    _, places, _ = step_and_diff([bn.StepEntry(s, [9 + i], [0]) for i, s in enumerate((c, b, e))])
    assert places == want([c, b, e])
    assert int((g4.tables_np[0, 2, 2:] != 0).sum()) == 0 and int((g4.tables_np[0, 3] != 0).sum()) == 0
    eng.cache.check()


def test_decode_steps_of_many_sequences_are_replayed_from_graphs(model_folders):
    """300 sequences decode together: more than the largest captured step holds (256 rows), so the step is replayed in
    two pieces (256 rows and 48 rows for the other 44); then 70 of them go on (a captured step of 96 rows).  float32:
    equal, bit for bit, to an engine that runs every step without graphs."""
    import bitnet_c_amd as bn
    folder = model_folders("A", torch.float32)
    reqs = _requests(256, 91, [1 + i % 9 for i in range(300)])
    outs = []
    for graphs in (True, False):
        eng = bn.Engine.from_folder(folder, dtype=torch.float32, max_tokens=64 * 320, use_graphs=graphs)
        slots = [eng.new_sequence() for _ in reqs]
        got = [eng.step([bn.StepEntry(s, r, [len(r) - 1]) for s, r in zip(slots, reqs)])]
        for k in range(2):
            got.append(eng.step([bn.StepEntry(s, [(7 * i + k) % 256], [0]) for i, s in enumerate(slots)]))
        for s in slots[70:]:
            eng.release(s)
        for k in range(2):
            got.append(eng.step([bn.StepEntry(s, [(5 * i + k) % 256], [0]) for i, s in enumerate(slots[:70])]))
        eng.cache.check()
        outs.append(got)
        if graphs:
            assert set(eng._graphs) == {256, 48, 96}
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_decode_step_takes_its_tokens_from_the_device(model_folders, dtype, graphs):
    """Tokens that a sampling kernel has left on the device are consumed from there: the same logits, bit for bit, as
    a step that is given the same tokens by the host; 300 sequences are more than one captured step holds, so the
    tensor is cut with the step.  A wrong tensor is refused and changes nothing."""
    import bitnet_c_amd as bn
    from bitnet_c_amd import ops
    from bitnet_c_amd.engine import StepError
    folder = model_folders("B", dtype)
    for n in (5, 300):
        reqs = _requests(389, 17 + n, [1 + i % 11 for i in range(n)])
        outs = []
        for on_device in (False, True):
            eng = bn.Engine.from_folder(folder, dtype=dtype, max_tokens=64 * (n + 4), use_graphs=graphs)
            slots = [eng.new_sequence() for _ in reqs]
            lg = eng.step([bn.StepEntry(s, r, [len(r) - 1]) for s, r in zip(slots, reqs)])
            got = []
            for k in range(3):
                toks = ops.argmax(lg)
                if on_device:
                    lg = eng.step([bn.StepEntry(s, [0], [0]) for s in slots], device_tokens=toks)
                else:
                    lg = eng.step([bn.StepEntry(s, [t], [0]) for s, t in zip(slots, toks.tolist())])
                got.append(lg)
                if k == 1:                      # the batch shrinks: rows of the token tensor are picked on the device
                    slots, lg = slots[1::2], lg[1::2].contiguous()
            if on_device:
                good = ops.argmax(lg)
                for bad, entries in ((good.to(torch.int64), None), (good[:-1], None), (good.cpu(), None),
                                     (good, [bn.StepEntry(s, [0, 1], [0]) for s in slots])):
                    with pytest.raises(StepError):
                        eng.step(entries or [bn.StepEntry(s, [0], [0]) for s in slots], device_tokens=bad)
                assert all(eng.length(s) == len(r) + 3 for s, r in zip(slots, reqs[1::2]))
            eng.cache.check()
            outs.append(got)
        for a, b in zip(*outs):
            assert torch.equal(a, b)


@pytest.mark.parametrize("n_tokens", [2048, 2000, 128])
def test_graph_replays_of_a_prompt_step_at_the_benchmark_layer_sizes(n_tokens):
    """A prompt step at the Llama-3.1-8B layer sizes (two layers, bfloat16) recorded into a graph: its products are the
    library's at their real sizes (the kernel the library picks for 2,048 rows of the feed-forward splits its work over
    the chip and keeps partial results in a work buffer), and a node that clears such a buffer inside a graph has to
    give the right result on every replay, not only on the first.  The same prompt in a new slot five times, other
    prompt steps and synchronisations between; the first run is eager, the second is the capture, the rest are replays;
    each is compared with the plain run of an engine that records nothing."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors
    raw = dict(model_type="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    model = DecoderModel(plan, torch.bfloat16, "cuda:0")
    model.load(random_tensors(plan.expected_tensors(), 3, torch.bfloat16, device="cuda:0"))
    engines = [bn.Engine(model, max_tokens=8192, max_seq_len=4096) for _ in range(2)]
    engines[1].prompt_graphs = False
    rnd = random.Random(41)
    toks = [rnd.randrange(cfg.vocab_size) for _ in range(n_tokens)]
    other = [rnd.randrange(cfg.vocab_size) for _ in range(700)]
    want = list(range(n_tokens - 4, n_tokens))

    def run(eng):
        s = eng.new_sequence()
        out = eng.step([bn.StepEntry(s, toks, want)])
        eng.release(s)
        return out

    ref = run(engines[1])
    rms = float(ref.double().pow(2).mean().sqrt())
    for k in range(5):
        got = run(engines[0])
        d = (got - ref).double()
        # the same kernels on the same rows: at most the rounding of a product whose sums the library forms in another order
        assert float(d.pow(2).mean().sqrt()) / rms < 0.01, k
        assert float(d.abs().max()) / rms < 0.1, k
        s = engines[0].new_sequence()                    # eager work of another size and a synchronisation between the replays
        engines[0].step([bn.StepEntry(s, other[:300 + 100 * k], [0])])
        engines[0].release(s)
        torch.cuda.synchronize()
    assert len(engines[0]._prompt_graphs) >= 1 and not engines[1]._prompt_graphs
    for e in engines:
        e.cache.check()


@pytest.mark.parametrize("n_seqs", [20, 50])
def test_graph_replays_of_a_wide_batch_at_the_benchmark_layer_sizes(n_seqs):
    """20 or 50 sequences decode together at the Llama-3.1-8B layer sizes (two layers, bfloat16): 32 or 64
    rows a step, whose products are the library's, replayed from a HIP graph.  A library kernel may clear a
    work buffer inside the graph, and such a node has to give the right result on every replay, not
    only on the first: every replay is compared with the same step run without graphs, with eager
    prompt steps of other sequences and synchronisations between the replays."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors
    raw = dict(model_type="llama", vocab_size=32000, hidden_size=4096, intermediate_size=14336,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               max_position_embeddings=8192, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    model = DecoderModel(plan, torch.bfloat16, "cuda:0")
    model.load(random_tensors(plan.expected_tensors(), 5, torch.bfloat16, device="cuda:0"))
    engines = [bn.Engine(model, max_tokens=64 * 160, use_graphs=g) for g in (True, False)]
    rnd = random.Random(41)
    reqs = [[rnd.randrange(cfg.vocab_size) for _ in range(10 + 3 * i)] for i in range(n_seqs)]
    extra = [[rnd.randrange(cfg.vocab_size) for _ in range(40)] for _ in range(6)]
    outs = []
    for eng in engines:
        slots = [eng.new_sequence() for _ in reqs]
        eng.step([bn.StepEntry(s, r[:-6], []) for s, r in zip(slots, reqs)])
        got = []
        for k in range(6):
            other = eng.new_sequence()                              # eager work between the replays
            eng.step([bn.StepEntry(other, extra[k], [39])])
            eng.release(other)
            torch.cuda.synchronize()
            got.append(eng.step([bn.StepEntry(s, [r[len(r) - 6 + k]], [0]) for s, r in zip(slots, reqs)]).clone())
        for s in slots:
            eng.release(s)
        eng.cache.check()
        outs.append(torch.stack(got))                               # [replay, sequence, vocab]
    assert engines[0]._graphs, "the decode steps were meant to be replayed from a graph"
    # The graph pads the batch to 32 or 64 rows and the library may pick another kernel for that many rows than for
    # 20 or 50, so the two sides differ by bfloat16 rounding: about 1 % of the logits' root mean square in every
    # row of every replay, with no value far outside it.  A buffer that was not cleared on a replay is not noise.
    rms = float(outs[1].double().pow(2).mean().sqrt())
    for k in range(6):
        d = (outs[0][k] - outs[1][k]).double()
        per_row = d.pow(2).mean(dim=1).sqrt() / rms
        assert float(per_row.max()) < 0.025, (k, per_row)
        # No single value far outside the noise.  Where most kernels are the same on both sides (only the attention's
        # split plan differs: the graph cuts for the longest sequence the engine allows) most differences are zero and
        # the measured deviation says nothing, so the yardstick is never smaller than what rounding gives at this
        # width when every kernel differs, 1.25 % of the logits' root mean square.
        sd = max(float(d.pow(2).mean().sqrt()), 0.0125 * rms)
        assert float(d.abs().max()) / sd < 8.0, k


# Further sizes than the tiny configurations': head sizes in steps of 16 up to 256, one to 64 heads in groups of 1 to 16,
# widths and vocabularies that are no power of two (some no multiple of 8), one to three layers, both rope forms, tied and
# untied, with and without biases; (head size, heads, kv heads, hidden, intermediate, vocab, layers, tied, biases, llama3
# scaling, prompt lengths)
FURTHER_SIZES = [
    (112, 16, 4, 264, 264, 256, 1, False, False, False, [7, 33, 33, 33, 70]),
    (112, 16, 1, 120, 520, 389, 2, True, False, False, [7, 70, 7, 70, 7, 19, 19, 19, 130, 7, 2, 2, 100, 1, 130, 7, 70, 70, 33, 100]),
    (256, 3, 3, 72, 172, 1000, 3, False, False, True, [1, 2, 130]),
    (96, 10, 2, 120, 1000, 389, 3, True, True, True, [19, 33, 100, 7, 100, 100, 130, 19, 19, 130, 1, 33, 33, 130, 130, 70, 2, 2, 19, 130]),
    (80, 64, 8, 64, 328, 97, 3, True, False, False, [2, 1, 70, 7, 33, 19, 7, 7, 1, 130, 1, 19, 100, 7, 130, 2, 2, 33, 100, 19]),
    (160, 4, 4, 72, 264, 2053, 3, True, False, True, [100]),
    (16, 4, 4, 136, 1000, 256, 1, False, False, True, [33, 33, 7, 33, 2, 2, 130, 19, 2, 130, 2, 130, 7, 2, 70, 100, 19, 2, 130, 19]),
    (48, 16, 8, 100, 173, 131, 2, False, False, False, [1, 40, 17]),
    # head sizes that are even and no multiple of 8 (rows of the cache that are no whole 16-byte groups)
    (20, 3, 3, 60, 100, 101, 2, False, False, True, [1, 40, 17, 70]),
    (36, 4, 2, 72, 173, 131, 1, True, False, False, [33, 2, 100]),
    (6, 6, 1, 30, 50, 61, 2, False, True, False, [5, 64, 65]),
    # forty heads of 128 with a kv head each (no grouping: one useful column in a tile of the matrix cores)
    (128, 40, 40, 160, 264, 389, 2, False, False, False, [200, 7, 130, 70, 33, 19, 100, 65]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act,F", [("gelu_pytorch_tanh", 264), ("relu2", 264), ("relu2", 173)])
def test_other_gate_activations_through_the_engine(tmp_path, act, F, dtype):
    """config.json's hidden_act reaches the feed-forward part as a parameter and the kernels as an argument:
    prompts (the library's product and the gated-unit kernel, or the float32 kernels), then decoded tokens (the
    streaming product's epilogue, with the norm folded in where the width allows), against the plain implementation."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.config import Architecture, ConfigError, register_architecture
    from bitnet_c_amd.config.llama import HIDDEN_ACTS
    from bitnet_c_amd.config.llama_plan import build_llama_plan

    # this architecture's config.json takes silu alone; another architecture of the family declares what it takes
    class OtherGateConfig(bn.LlamaConfig):
        GATE_ACTIVATIONS = tuple(HIDDEN_ACTS)

    register_architecture(Architecture("other_gate_test", OtherGateConfig, build_llama_plan), replace=True)
    raw = dict(model_type="other_gate_test", vocab_size=211, hidden_size=128, intermediate_size=F, num_hidden_layers=2,
               num_attention_heads=4, num_key_value_heads=2, head_dim=32, max_position_embeddings=512,
               rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False, hidden_act=act)
    with pytest.raises(ConfigError, match="hidden_act"):
        bn.LlamaConfig.from_dict(dict(raw, model_type="llama"))
    folder = bn.write_model_folder(str(tmp_path / "m"), OtherGateConfig.from_dict(raw), 77, dtype)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    assert c["act"] == act
    eng = bn.Engine.from_folder(folder, dtype=dtype, max_tokens=1024)
    assert eng.model.blocks[0].ffn.activation == {"gelu_pytorch_tanh": "gelu_tanh", "relu2": "relu2"}[act]
    reqs = _requests(211, 78, [37, 74, 9])
    slots = [eng.new_sequence() for _ in reqs]
    got = [[] for _ in reqs]
    lg = eng.step([bn.StepEntry(s, r[:-4], list(range(len(r) - 4))) for s, r in zip(slots, reqs)])
    at = 0
    for i, r in enumerate(reqs):
        got[i].append(lg[at:at + len(r) - 4])
        at += len(r) - 4
    for t in range(4):
        lg = eng.step([bn.StepEntry(s, [r[len(r) - 4 + t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(lg[i:i + 1].clone())
    rounded = torch.bfloat16 if dtype == torch.bfloat16 else None
    for i, r in enumerate(reqs):
        want = pl.forward(c, W, r, rounded)
        assert rel_err(torch.cat(got[i]), want) < TOL[dtype], i
        other = pl.forward(dict(c, act="silu"), W, r, rounded)           # and it is not the default activation's result
        assert rel_err(other, want) > 2 * TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(FURTHER_SIZES)))
def test_further_sizes(tmp_path, case, dtype):
    """Unequal prompts in one step (logits at every place), then four tokens each, at sizes that the other tests
    do not have; against the plain implementation."""
    import bitnet_c_amd as bn
    hs, H, Hkv, hidden, F, V, L, tied, biases, scaling, lens = FURTHER_SIZES[case]
    raw = dict(model_type="llama", vocab_size=V, hidden_size=hidden, intermediate_size=F, num_hidden_layers=L,
               num_attention_heads=H, num_key_value_heads=Hkv, head_dim=hs, max_position_embeddings=1024,
               rope_theta=500000.0 if scaling else 10000.0, rms_norm_eps=1e-6 if tied else 1e-5,
               tie_word_embeddings=tied, attention_bias=False, mlp_bias=biases)
    if scaling:
        raw["rope_scaling"] = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                   original_max_position_embeddings=64)
    folder = bn.write_model_folder(str(tmp_path / "m"), bn.LlamaConfig.from_dict(raw), 100 + case, dtype)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    eng = bn.Engine.from_folder(folder, dtype=dtype, max_tokens=max(2048, 64 * 4 * len(lens)))
    n_dec = 4
    reqs = _requests(V, 200 + case, [n + n_dec for n in lens])
    slots = [eng.new_sequence() for _ in reqs]
    got = [[] for _ in reqs]
    lg = eng.step([bn.StepEntry(s, r[:-n_dec], list(range(len(r) - n_dec))) for s, r in zip(slots, reqs)])
    at = 0
    for i, r in enumerate(reqs):
        got[i].append(lg[at:at + len(r) - n_dec])
        at += len(r) - n_dec
    for t in range(n_dec):
        lg = eng.step([bn.StepEntry(s, [r[len(r) - n_dec + t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(lg[i:i + 1].clone())
    for s in slots:
        eng.release(s)
    eng.cache.check()
    for i, r in enumerate(reqs):
        want = pl.forward(c, W, r, torch.bfloat16 if dtype == torch.bfloat16 else None)
        assert rel_err(torch.cat(got[i]), want) < TOL[dtype], (i, len(r))
