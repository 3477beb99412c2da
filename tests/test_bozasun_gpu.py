"""The Bozasun decoder through the engine against the plain implementation: whole prompts, decoding through
cache and state, portions down to two tokens, unequal batches, slots and pages used again, sizes of several
kinds, keys just inside and just outside a chunk of positions (in prompts and in decoding, at the pages' edges),
far keys and long memories, the first tokens of a sequence, greedy generation through the entry point, the trace
program and the command line; float32 and bfloat16."""
import numpy as np
import pytest
import torch

import herbert_rs_amd as hb
from herbert_rs_amd.engine import StepEntry

from . import replay_util as ru
from .bounds import close
from .bozasun_tiny import CONFIGS, make_folder, plain_folder, plain_logits, random_tokens
from .plain import bozasun as plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]

# In bfloat16 the router sees rows that differ from the plain ones by their rounding, and of a few hundred
# choices among close scores some fall the other way: such a token then runs through another expert, which no
# bound on rounding covers, and the keys and the state of later layers carry it on to later tokens. Float32 is
# compared row by row without exception. In bfloat16 a share of the rows may be off where experts are chosen
# (the mechanisms alone, where nothing is chosen, are held to the rounding of their kernels in
# test_bozasun_kernels_gpu.py); where every layer is dense or every expert runs, one row in twenty-five may pass
# the bound: the norm behind the state-space layer's gate divides by the root mean square of a row that is now and
# then small, which multiplies the rounding that the row's input carries (forty times on a row of a layer with one
# head and one norm group, in the engine as in the plain formulas when their inputs are rounded to bfloat16); such
# a row stays below half the logits' own size, which a fault of cache, state or batch does not.
FLIPPED_SHARE = 0.25
TAIL_SHARE, TAIL_LIMIT = 0.04, 0.5


def chooses(raw):
    for l in raw["layers"]:
        m = l["mlp"]
        if m is not None and m["kind"] == "moe" and m["router"]["top"] < m["router"]["experts"] + m["router"].get("identity", 0):
            return True
    return False


def compare(rows, folder, tokens, positions, dtype, label, raw=None):
    ref = plain_logits(folder, tokens)
    raw = raw if raw is not None else CONFIGS[label.split()[0]][0]
    off = []
    for row, p in zip(rows, positions):
        assert np.isfinite(np.asarray(row)).all(), f"{label}: position {p} is not finite"
        ok, err = close(np.asarray(row), ref[p], dtype, "boz", label)
        if not ok:
            off.append((p, err))
    n = len(list(positions))
    if dtype == "float32":
        assert not off, f"{label}: positions and errors {off[:5]}"
    elif not chooses(raw):
        assert len(off) <= max(2, TAIL_SHARE * n) and all(e <= TAIL_LIMIT for _, e in off), \
            f"{label}: positions and errors {off[:5]}"
    else:
        assert len(off) <= max(3, FLIPPED_SHARE * n), f"{label}: {len(off)} of {n} rows off: {off[:5]}"


def feed(engine, slot, tokens, cuts):
    """The tokens of one sequence in portions that end at `cuts`; every position's logits, in order."""
    rows, at = [], 0
    for end in list(cuts) + [len(tokens)]:
        if end <= at:
            continue
        part = tokens[at:end]
        rows.append(engine.step([StepEntry(slot, part, list(range(len(part))))]).cpu().numpy())
        at = end
    return np.concatenate(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_whole_prompts_and_token_by_token(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for n, seed in ((1, 1), (2, 2), (3, 6), (67, 3), (150, 4)):
        tokens = random_tokens(vocab, n, seed)
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, []), folder, tokens, range(n), dtype, f"{name} whole")
        engine.free_slot(slot)
    # the first tokens of a sequence one by one, then on through a page's edge and several chunks' edges: the
    # states of a fresh slot, the filter's empty past, a chunk's first key alone in its softmax
    tokens = random_tokens(vocab, 140, 5)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, range(1, 140)), folder, tokens, range(140), dtype, f"{name} one by one")
    engine.free_slot(slot)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "S"])
def test_portions_of_several_sizes_and_slots_used_again(name, dtype, model_root):
    """Portions shorter than the filter's taps, portions that end beside a page's edge and beside a chunk's, and
    one long one; every pass takes the slot and pages that the pass before gave back."""
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=512)
    tokens = random_tokens(vocab, 200, 21)
    for cuts in ([2, 4, 7], [64, 128], [63, 65, 127, 129, 192], [1, 3, 49, 50, 51, 100, 102, 199], [150]):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(200), dtype, f"{name} portions")
        engine.free_slot(slot)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_unequal_batches_against_each_alone(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    lengths = [1, 90, 33, 140, 64, 2]
    seqs = [random_tokens(vocab, n + 12, 40 + i) for i, n in enumerate(lengths)]
    for again in range(2):               # twice: the second time the slots and pages were used before
        slots = [engine.alloc_slot() for _ in seqs]
        out = engine.step([StepEntry(s, t[:n], list(range(n))) for s, t, n in zip(slots, seqs, lengths)]).cpu().numpy()
        at = 0
        for t, n in zip(seqs, lengths):
            compare(out[at:at + n], folder, t, range(n), dtype, f"{name} batch prompts")
            at += n
        live = list(range(len(seqs)))
        for step in range(12):
            if step == 5:                # a sequence ends early; its slot goes back while the others go on
                engine.free_slot(slots[live.pop(1)])
            out = engine.step([StepEntry(slots[i], [seqs[i][lengths[i] + step]], [0]) for i in live]).cpu().numpy()
            for row, i in zip(out, live):
                compare([row], folder, seqs[i], [lengths[i] + step], dtype, f"{name} batch decode")
        for i in live:
            engine.free_slot(slots[i])
        engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_of_a_batch(dtype, model_root):
    """Several sequences go on by portions of unequal sizes in the same steps: every sequence's filter, state and
    chunks continue from its own slot and its own positions."""
    folder = make_folder(model_root, "P", dtype)
    vocab = CONFIGS["P"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    seqs = [random_tokens(vocab, n, 140 + i) for i, n in enumerate([130, 71, 9])]
    slots = [engine.alloc_slot() for _ in seqs]
    at = [0, 0, 0]
    for sizes in ([2, 64, 1], [62, 1, 2], [3, 2, 3], [63, 4, 3]):
        entries, spans = [], []
        for i, n in enumerate(sizes):
            part = seqs[i][at[i]:at[i] + n]
            entries.append(StepEntry(slots[i], part, list(range(len(part)))))
            spans.append((i, at[i], len(part)))
            at[i] += len(part)
        out = engine.step(entries).cpu().numpy()
        row = 0
        for i, first, n in spans:
            compare(out[row:row + n], folder, seqs[i], range(first, first + n), dtype, "P portions of a batch")
            row += n


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype, model_root):
    """300 tokens one by one: the decode steps replayed as graphs, the pages' edges, two chunks' edges, the state
    and the filter's last inputs carried on."""
    folder = make_folder(model_root, "Q", dtype)
    vocab = CONFIGS["Q"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=512)
    tokens = random_tokens(vocab, 330, 77)
    slot = engine.alloc_slot()
    compare(feed(engine, slot, tokens, [30] + list(range(31, 330))), folder, tokens, range(330), dtype, "Q long decode")
    engine.free_slot(slot)


def _sharp_folder(model_root, dtype):
    """F with scores made sharp (queries' and keys' norm weights scaled up: a score's cap is 40, so a few keys hold
    a query's weight) and the state-space layer's decay near one (exp(A_log) small), so that its state remembers
    the sequence's start."""
    return make_folder(model_root, "F", dtype, set_to={".mix.A_log": -6.0}, tag="_long")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_and_a_long_memory_show(dtype, model_root):
    """The logits depend on tokens hundreds back, in the prompt and in decoding, across the pages' edges (the
    attention without chunks, the latent attention, the state): checked on the plain implementation, then the
    engine against it."""
    folder = _sharp_folder(model_root, dtype)
    vocab = CONFIGS["F"][0]["vocab"]
    tokens = random_tokens(vocab, 400, 91)
    cfg, w = plain_folder(folder)
    a = plain_logits(folder, tokens)[-1]
    for changed in (3, 70):
        other = list(tokens)
        other[changed] = (other[changed] + 1) % vocab
        b = plain.forward(cfg, w, other, rows=[399])[0].numpy()
        assert np.abs(a - b).max() > 0.005 * np.abs(a).max(), f"token {changed} does not show in the plain logits"
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for cuts in ([], [128, 256], [360] + list(range(361, 400))):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(400), dtype, "F far")
        engine.free_slot(slot)


class EdgeModel:
    """One attention layer whose scores are sharp (the queries' norm weights are scaled up until most scores sit
    near the cap, plus or minus), so that a few keys hold a query's weight and a key that is wrongly seen, or
    wrongly missed, at a chunk's edge moves the logits. (The kernels' test makes single keys stand out by hand.)"""

    def __init__(self, chunk, softcap=None):
        from .bozasun_tiny import attention, dense, model, rot
        self.raw = model(64, 64, [attention(2, 1, 32, 32, 0.5, rot(32, 100.0, 2.0), chunk=chunk, softcap=softcap, mlp=dense(64))],
                         eps=1e-5)
        self.chunk = chunk

    def folder(self, root, dtype):
        folder = str(root / f"edge_{self.chunk}_{dtype}")
        hb.write_random_model(folder, self.raw, seed=7, dtype=dtype, std=0.1, norm_std=0.1)
        import os
        from safetensors import safe_open
        from safetensors.torch import save_file
        path = os.path.join(folder, "model.safetensors")
        with safe_open(path, framework="pt") as f:
            tensors = {k: f.get_tensor(k) for k in f.keys()}
        tensors["l0.mix.q.norm"] = (tensors["l0.mix.q.norm"].float() * 8.0).to(tensors["l0.mix.q.norm"].dtype)
        save_file(tensors, path)
        return folder


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [7, 64, 100])
def test_keys_just_inside_and_just_outside_a_chunk(chunk, dtype, tmp_path):
    """Every position's logits around the edges of chunks of 7, 64 (a page) and 100 positions: whole, with portions
    that end on, before and after an edge, and one token at a time. That a key on the other side of an edge would
    show is checked on the plain implementation: with chunks one position longer the rows behind an edge move."""
    em = EdgeModel(chunk, softcap=10.0)
    folder = em.folder(tmp_path, dtype)
    tokens = random_tokens(64, 3 * chunk + 5 if chunk > 7 else 80, 12)
    n = len(tokens)
    ref = plain_logits(folder, tokens)
    cfg, w = plain_folder(folder)
    longer = {**cfg, "layers": [{**cfg["layers"][0], "mixer": {**cfg["layers"][0]["mixer"], "mask": {"size": chunk + 1}}}]}
    moved = plain.forward(longer, w, tokens).numpy()
    edge = 2 * chunk
    assert np.abs(moved[edge] - ref[edge]).max() > 0.02 * np.abs(ref[edge]).max()
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    for cuts in ([], [chunk], [chunk - 1, chunk + 1, 2 * chunk - 1], [2 * chunk + 1], list(range(chunk - 2, min(n, 2 * chunk + 3)))):
        slot = engine.alloc_slot()
        compare(feed(engine, slot, tokens, cuts), folder, tokens, range(n), dtype, f"edge {chunk}", raw=em.raw)
        engine.free_slot(slot)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_layers(dtype, model_root):
    """Heads of 128, a state of 128 rows, a latent of 256 + 32, experts of 256: the sizes of a larger model's layers."""
    folder = make_folder(model_root, "W", dtype)
    vocab = CONFIGS["W"][0]["vocab"]
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    tokens = random_tokens(vocab, 300, 5)
    rows = [0, 1, 2, 3, 63, 64, 100, 126, 127, 128, 191, 192, 193, 255, 256, 279]
    slot = engine.alloc_slot()
    out = engine.step([StepEntry(slot, tokens[:280], rows)]).cpu().numpy()
    compare(out, folder, tokens, rows, dtype, "W prompt")
    for p in range(280, 300):
        out = engine.step([StepEntry(slot, [tokens[p]], [0])]).cpu().numpy()
        compare(out, folder, tokens, [p], dtype, "W decode")
    engine.free_slot(slot)


def drawn_configuration(seed):
    """A configuration whose sizes, options and order of layers are drawn: widths and vocabularies that are no
    powers of two, keys of 24 to 160 and values of 16 to 144, 1 to 12 heads, chunks of 5 to 200 positions or none,
    capped scores or not, rotation of a part or of the whole head or none, slowed or not, latents of 24 to 256 with
    rotated parts of 4 to 64, states of 8 to 128 rows, 1 to 4 taps, experts with and without groups and identity
    experts, feed-forwards present or not, a token input or none."""
    import random
    from .bozasun_tiny import attention, dense, latent, mamba, model, moe, rot
    r = random.Random(seed)
    width = r.choice([64, 96, 136, 160, 200, 256, 320])

    def mlp():
        kind = r.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return dense(r.choice([48, 100, 192, 320]))
        identity = r.choice([0, 0, 1, 2, 4])
        experts = r.choice([2, 3, 4, 6, 8])
        total = experts + identity
        groups = None
        divisors = [c for c in (2, 3, 4) if total % c == 0]
        if divisors and r.random() < 0.6:
            count = r.choice(divisors)
            groups = (count, r.randint(1, count))
        room = total if groups is None else groups[1] * (total // groups[0])
        return moe(r.choice([24, 32, 64, 96]), experts, r.randint(1, min(room, 4)), identity, groups)

    layers = []
    for _ in range(r.randint(1, 4)):
        kind = r.choice(["attention", "latent", "mamba"])
        if kind == "attention":
            kv = r.choice([1, 2, 4])
            dim, vdim = r.choice([24, 32, 48, 64, 80, 128, 160]), r.choice([16, 40, 64, 80, 128, 144])
            dims = r.choice([dim, dim, 2 * (dim // 4), 8])
            rotation = r.choice([None, rot(dims, r.choice([20.0, 10000.0]), r.choice([None, 2.0, 8.0]))])
            layers.append(attention(kv * r.choice([1, 2, 3]), kv, dim, vdim, r.choice([0.5, 1.0]) * dim ** -0.5, rotation,
                                    r.choice([None, 5, 32, 50, 64, 200]), r.choice([None, 5.0, 30.0]), mlp()))
        elif kind == "latent":
            rd = r.choice([4, 8, 16, 32, 64])
            dim = r.choice([16, 24, 32, 64])
            layers.append(latent(r.randint(1, 6), dim, rd, r.choice([16, 24, 32, 64]), r.choice([24, 32, 64, 96, 256]),
                                 (dim + rd) ** -0.5, r.choice([100.0, 10000.0]), mlp(), r.choice([None, None, 4.0])))
        else:
            groups = r.choice([1, 2, 3])
            heads = groups * r.choice([1, 2, 4])
            vdim = r.choice([8, 16, 32, 40, 64])
            ng = r.choice([g for g in (1, 2, 4) if (heads * vdim) % g == 0])
            layers.append(mamba(heads, vdim, r.choice([8, 16, 24, 64, 128]), groups, r.randint(1, 4), ng, mlp()))
    return model(r.choice([100, 257, 448, 600]), width, layers, eps=r.choice([1e-6, 1e-5, 3e-5]), side=r.choice([None, 1, 7, 16, 48]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations(seed, dtype, tmp_path):
    """Sixteen drawn configurations: a prompt whole, decoded on, and beside a second request in portions and single
    tokens. (A one-off sweep of 80 further draws had six beyond the bounds, none of them a fault: three float32 rows
    of stacks of state-space layers at 1.1e-4 to 5e-4, the rows at which the plain formulas in float32 are themselves
    7e-5 to 9e-5 from their float64 (the norm behind the gate divides by a root mean square that is small there);
    two bfloat16 draws with norm groups of 4 and 10 channels; and one whose only expert of a token fell the other
    way at position 5, which the states of the layers behind carried on for a few tokens more than the share
    allows.)"""
    raw = drawn_configuration(seed)
    folder = str(tmp_path / "drawn")
    hb.write_random_model(folder, raw, seed=100 + seed, dtype=dtype, std=0.1, norm_std=0.1)
    vocab = raw["vocab"]
    a, b = random_tokens(vocab, 150, 300 + seed), random_tokens(vocab, 40, 400 + seed)
    engine = hb.load(folder, dtype=dtype, cache_tokens=1024)
    label = f"drawn {seed}"
    slot = engine.alloc_slot()
    compare(feed(engine, slot, a, [131] + list(range(132, 150))), folder, a, range(150), dtype, label, raw=raw)
    engine.free_slot(slot)
    sa, sb = engine.alloc_slot(), engine.alloc_slot()
    out = engine.step([StepEntry(sa, a[:70], list(range(70))), StepEntry(sb, b[:3], [0, 1, 2])]).cpu().numpy()
    compare(out[:70], folder, a, range(70), dtype, label, raw=raw)
    compare(out[70:], folder, b, range(3), dtype, label, raw=raw)
    for i in range(8):
        out = engine.step([StepEntry(sa, [a[70 + i]], [0]), StepEntry(sb, [b[3 + i]], [0])]).cpu().numpy()
        compare([out[0]], folder, a, [70 + i], dtype, label, raw=raw)
        compare([out[1]], folder, b, [3 + i], dtype, label, raw=raw)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(name, dtype, model_root):
    folder = make_folder(model_root, name, dtype)
    vocab = CONFIGS[name][0]["vocab"]
    cfg, w = plain_folder(folder)
    prompts = [random_tokens(vocab, n, 60 + n) for n in (9, 1, 70)]
    got = hb.generate(folder, prompts, temperature=0.0, max_tokens=10, ignore_eos=True, no_repeat_check=True, dtype=dtype)
    for p, g in zip(prompts, got):
        assert len(g) == 10
        if dtype == "float32":
            assert g == plain.greedy(cfg, w, p, 10)
            continue
        seq = list(p)                    # bfloat16 may flip a near-tie, or an expert: the token must then be close to the best
        far = 0
        for tok in g:
            logits = plain.forward(cfg, w, seq, rows=[len(seq) - 1])[0]
            far += float(logits.max() - logits[tok]) > 0.05 * float(logits.std()) + 1e-6
            seq.append(tok)
        assert far <= 2


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program(dtype, model_root, tmp_path):
    folder = make_folder(model_root, "P", dtype)
    vocab = CONFIGS["P"][0]["vocab"]
    reqs = {f"r{i}": random_tokens(vocab, n, 200 + i) for i, n in enumerate([5, 130, 1, 66, 40])}
    for label, steps in (("whole", ru.trace_whole(reqs)), ("tail", ru.trace_tail(reqs, 20)),
                         ("batches", ru.trace_batches(reqs, 3, 0.6))):
        held = max(sum(len(t) for t in reqs.values()), 1)
        out = ru.run_trace(folder, dtype, steps, str(tmp_path / label), held, vocab)
        got = ru.collect(steps, out)
        assert len(got) == sum(len(t) for t in reqs.values())
        by_request = {}
        for (rid, pos), row in got.items():
            by_request.setdefault(rid, []).append((pos, row))
        for rid, rows in by_request.items():
            rows.sort(key=lambda pr: pr[0])
            compare([r for _, r in rows], folder, reqs[rid], [p for p, _ in rows], dtype, f"P trace {label}")


def test_the_command_line_generates_token_ids(model_root):
    """The command line serves the family as it serves any other: token ids in, token ids out (--max-tokens 6 gives
    seven tokens: it counts the decode steps after the prompt's own token), with sampling parameters too."""
    import os
    import subprocess
    import sys
    folder = make_folder(model_root, "P", "float32")
    cfg, w = plain_folder(folder)
    cli = os.path.join(ru.ROOT, "bin", "herbert-cli")
    out = subprocess.run([sys.executable, cli, "--model", folder, "--prompt", "5,17,3,190", "--temperature", "0",
                          "--max-tokens", "6", "--dtype", "float32", "--ignore-eos", "--no-repeat-check", "--verbose"],
                         capture_output=True, text=True, timeout=240)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.strip().split(",")] == plain.greedy(cfg, w, [5, 17, 3, 190], 7)
    drawn = [subprocess.run([sys.executable, cli, "--model", folder, "--prompt", "5,17,3,190", "--temperature", "0.8",
                             "--top-k", "20", "--top-p", "0.9", "--seed", "3", "--max-tokens", "6", "--dtype", "float32",
                             "--ignore-eos", "--no-repeat-check"], capture_output=True, text=True, timeout=240)
             for _ in range(2)]
    assert all(d.returncode == 0 for d in drawn), drawn[0].stderr
    assert drawn[0].stdout == drawn[1].stdout and len(drawn[0].stdout.strip().split(",")) == 7
