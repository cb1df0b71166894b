"""The step's tables and the attention kernels' launch shapes, on the host.

The table builder (``ModelRunner.step_tables``), the attention planner and the
cache manager need no device: this file builds a runner over pools that hold no
memory and checks, for random eager and recorded ("fixed") steps, that every
index a kernel will form from the tables stays inside what was allocated.  The
index ranges of the attention kernels are re-derived here, workgroup by
workgroup, from the same formulas as csrc/kernels/attention.hip uses (grid
shapes, the unit a workgroup takes, the runs of keys, the partial-result
indices), so that a table or a launch shape that would send a kernel out of
bounds fails here and not on a GPU.
"""
import numpy as np
import pytest
import torch

from conftest import TINY_A, TINY_B, TINY_C

LLAMA_1B = dict(
    architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=2048, intermediate_size=8192,
    num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64, max_position_embeddings=8192,
    rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True)
LLAMA_8B_LAYER = dict(LLAMA_1B, hidden_size=4096, intermediate_size=14336, head_dim=128)


def runner_on_host(raw, pages, page_size, slots=8, dtype=torch.bfloat16):
    """A step function without a device: model structure, cache manager, pools on the meta device."""
    from lyapunov_engine_amd.cache.manager import CacheManager, CachePools, GroupConfig
    from lyapunov_engine_amd.config import LlamaConfig
    from lyapunov_engine_amd.engine.runner import ModelRunner
    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.models.llama import llama_spec

    cfg = LlamaConfig.from_dict(raw)
    model = build_model(llama_spec(cfg))
    model.max_positions = min(cfg.max_position_embeddings, pages * page_size)
    layout = model.cache_layout()
    groups = [GroupConfig(pages, page_size, gl.spec.window) for gl in layout.groups]
    cache = CacheManager(groups, slots)
    pools = CachePools(layout, groups, slots, dtype, "meta")
    return ModelRunner(model, cache, pools, dtype, "cpu"), cfg


def sections(t):
    out = {}
    for name, off, size in zip(t.names, t.offsets, t.sizes):
        out[name] = t.host[off:off + size]
    return out


# ------------------------------------------------ the kernels' index ranges, re-derived
WIDE_KEYS = lambda hd: 64 if hd <= 64 else 32       # WideTile::kKeys


def prefill_ranges(sec, launch, *, nh, nkv, hd, bs, width, wide, n_pages, T, units_of_device=256):
    """Walk the workgroups of lyp_attn_prefill's launch over these tables and assert that every
    table index, page, token row and partial-result index they form is inside its array.
    Returns the number of workgroups that found work."""
    q_start, ctx_len = sec["q_start"], sec["ctx_len"]
    tile_seq, tile_q0 = sec[("plan", KEY, "tile_seq")], sec[("plan", KEY, "tile_q0")]
    table = sec[("block_table", 0)].reshape(-1, width)
    B = ctx_len.size
    n_tiles, parts = launch["n_tiles"], launch["parts"]
    assert tile_seq.size == n_tiles and tile_q0.size == n_tiles and 1 <= parts <= 16
    g = nh // nkv
    gh = 4 if g >= 4 else (2 if g >= 2 else 1)
    head_groups = -(-g // gh)
    if wide:
        nw = 4 if gh == 1 else 8
        qw = (nw // gh) * 16
    else:
        assert parts == 1
        qb = 2 if (gh == 4 and hd <= 64) else 1
        qw = (4 // gh) * qb * 16
    subs = 64 // qw
    units = n_tiles * subs
    wgs = units * nkv * head_groups * parts
    paired = wide and launch["pair"] and parts == 1 and wgs > units_of_device
    KT = WIDE_KEYS(hd) if wide else (64 if hd * 2 <= 128 else (32 if hd * 2 <= 256 else 16))
    busy = 0
    ys = (units + 1) // 2 if paired else units
    for y in range(ys):
        for rnd in range(2 if paired else 1):
            unit = units - 1 - y
            if rnd == 1:
                if 2 * y >= units - 1:
                    break
                unit = y
            tile = unit // subs
            assert 0 <= tile < n_tiles
            seq = int(tile_seq[tile])
            assert 0 <= seq < B, f"tile {tile} names request {seq} of {B}"
            tok0, q_len, ctx = int(q_start[seq]), int(q_start[seq + 1] - q_start[seq]), int(ctx_len[seq])
            q0 = int(tile_q0[tile]) + (unit % subs) * qw
            assert q0 >= 0
            if q0 >= q_len:
                continue
            busy += 1
            pos_first = ctx - q_len + q0
            assert pos_first >= 0, "a request brings more tokens than it is long"
            hi = pos_first + min(qw, q_len - q0)
            assert hi <= ctx <= width * bs
            assert tok0 + q0 + min(qw, q_len - q0) <= T                     # query and output rows
            blk_last = (hi - 1) // bs
            assert blk_last < width
            used = table[seq, :blk_last + 1]
            assert ((used >= -1) & (used < n_pages)).all(), f"request {seq}: a table entry outside the pool"
            if parts > 1:
                kt_base = 0
                run = -(-(-(-(hi - kt_base) // KT)) // parts) * KT
                for z in range(parts):
                    assert kt_base + z * run >= 0
                in_tile_most = q0 - int(tile_q0[tile]) + min(qw, q_len - q0) - 1
                assert 0 <= in_tile_most < 64
                pidx = ((tile * 64 + in_tile_most) * nh + nh - 1) * parts + parts - 1
                assert (pidx + 1) * hd <= launch["part_o"] and (pidx + 1) * 2 <= launch["part_ml"], \
                    "the runs' partial results do not fit their workspace"
    # the merge kernel: grid (nh, 64, n_tiles), reads tile_seq/tile_q0 of every tile, live or not
    for tile in range(n_tiles):
        seq = int(tile_seq[tile])
        assert 0 <= seq < B
    return busy


def decode_ranges(sec, launch, *, nh, nkv, hd, bs, width, n_pages, T, B, waves):
    """The same for lyp_attn_decode's launch: grid (max_parts, nkv * column groups, n_dec)."""
    q_start, ctx_len = sec["q_start"], sec["ctx_len"]
    dec = sec.get(("plan", KEY, "dec"))
    table = sec[("block_table", 0)].reshape(-1, width)
    n_dec, part_keys, max_parts = launch["n_dec"], launch["part_keys"], launch["max_parts"]
    assert part_keys % (waves * 64) == 0
    for slot in range(n_dec):
        seq = int(dec[slot]) if dec is not None else slot
        assert 0 <= seq < B
        ctx = int(ctx_len[seq])
        assert 0 <= ctx <= width * bs and int(q_start[seq]) < T
        # a request's partitions: every key has to fall into one of the max_parts workgroups
        most = part_keys // waves
        block = waves * most
        n_parts = max(1, -(-ctx // block))
        per_part = -(-ctx // n_parts) if ctx else 0
        kpw = max(16, -(-per_part // (waves * 16)) * 16)
        assert -(-ctx // (waves * kpw)) <= max_parts, f"request of {ctx} keys needs more than {max_parts} partitions"
        used = table[seq, :-(-ctx // bs)]
        assert ((used >= -1) & (used < n_pages)).all()
        pidx = (slot * nh + nh - 1) * max_parts + max_parts - 1
        assert (pidx + 1) * hd <= launch["part_o"] and (pidx + 1) * 2 <= launch["part_ml"]


# ------------------------------------------------------------------- random steps
def live_requests(rng, cache, rows, fixed_tokens, max_context, page_size):
    """Up to ``rows`` live requests for a fixed step: ids, starts, counts."""
    n = int(rng.integers(0, rows + 1))
    ids, starts, counts, left = [], [], [], fixed_tokens
    for i in range(n):
        if fixed_tokens:
            if left < 1:
                break
            count = int(rng.integers(1, left + 1)) if rng.random() < 0.7 else min(left, int(rng.choice([1, 2, 63, 64, 65])))
            left -= count
        else:
            count = 1
        start = int(rng.integers(0, max_context - count + 1))
        if rng.random() < 0.3:
            start = min(start // page_size * page_size + int(rng.choice([0, 1, page_size - 1])), max_context - count)
        rid = 100 + i
        if not cache.can_extend(rid, start + count):
            continue
        cache.add(rid)
        cache.extend(rid, start + count)
        cache.commit(rid, start)
        ids.append(rid), starts.append(start), counts.append(count)
    return (np.asarray(ids, dtype=np.int64), np.asarray(starts, dtype=np.int32), np.asarray(counts, dtype=np.int32))


from lyapunov_engine_amd.parts.attention import AttentionWork  # noqa: E402

KEY = AttentionWork.key

CASES = [("A", TINY_A, 4, False), ("B", TINY_B, 16, True), ("C", TINY_C, 16, True), ("1B", LLAMA_1B, 16, True),
         ("8B-layer", LLAMA_8B_LAYER, 16, True)]


@pytest.mark.parametrize("name,raw,page_size,wide", CASES, ids=[c[0] for c in CASES])
def test_recorded_steps_keep_every_index_inside_its_array(name, raw, page_size, wide):
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.base import FixedStep

    rng = np.random.default_rng(7)
    nh, nkv, hd = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
    none64, none32 = np.zeros(0, np.int64), np.zeros(0, np.int32)
    for trial in range(60):
        max_pos = raw["max_position_embeddings"]
        max_context = int(rng.choice([c for c in (256, 512, 1024, 2048, 4096, 8192) if c <= max_pos]))
        tokens = int(rng.choice([0, 16, 32, 64, 128, 256, 512]))
        tokens = min(tokens, max_context)
        rows = int(rng.integers(1, 5)) if tokens else int(rng.choice([1, 2, 3, 4, 6, 8, 16, 64]))
        # few pages: just enough for the step's bound, sometimes fewer than every row could ask for
        pages = max(-(-max_context // page_size) * int(rng.integers(1, 3)), 4)
        runner, cfg = runner_on_host(raw, pages, page_size, slots=max(rows, 4))
        runner.max_position = max_pos          # the tables' bound under test is the step's, not the pool's
        mixer = runner.model.layers[0].mixer
        fixed = FixedStep(rows=rows, max_context=max_context, tokens=tokens)
        empty = runner.step_tables(none64, none32, None, none32, None, fixed=fixed)
        ids, starts, counts = live_requests(rng, runner.cache, rows, tokens, max_context, page_size)
        toks = rng.integers(0, raw["vocab_size"], int(counts.sum()) if tokens else len(ids)).astype(np.int32)
        t = runner.step_tables(ids, starts, counts if tokens else None, toks, None, fixed=fixed)
        what = f"{name} trial {trial}: {fixed}, live {list(zip(ids.tolist(), starts.tolist(), counts.tolist()))}"
        assert t.shape_key() == empty.shape_key(), what
        sec = sections(t)
        T, B, n = t.T, t.B, len(ids)
        assert T == fixed.token_rows and B == rows
        width = t.widths[0]
        assert width == -(-max_context // page_size)
        q_start, ctx_len, pos = sec["q_start"], sec["ctx_len"], sec["positions"]
        assert q_start[0] == 0 and (np.diff(q_start) >= 0).all() and q_start[-1] <= T, what
        if not tokens:
            assert q_start[-1] == T
        live_tokens = int(q_start[n])
        assert (sec["token_ids"] >= 0).all() and (sec["token_ids"] < raw["vocab_size"]).all()
        assert (pos >= 0).all() and (pos < max_pos).all() and (ctx_len <= max_context).all()
        slots = sec[("slot_mapping", 0)]
        assert ((slots == -1) | ((slots >= 0) & (slots < pages * page_size))).all(), what
        assert (slots[:live_tokens] >= 0).all() and (slots[live_tokens:] == -1).all(), what
        assert len(set(slots[:live_tokens].tolist())) == live_tokens, "two tokens share a slot"
        table = sec[("block_table", 0)]
        assert ((table >= -1) & (table < pages)).all(), what
        assert (sec["state_slots"][n:] == runner.cache.num_state_slots).all()
        rows_wanted = sec["logit_rows"]
        assert rows_wanted.size == rows and (rows_wanted >= 0).all() and (rows_wanted < T).all()
        tile_seq, tile_q0 = sec[("plan", KEY, "tile_seq")], sec[("plan", KEY, "tile_q0")]
        count = np.diff(q_start)
        for s, q0 in zip(tile_seq, tile_q0):
            assert 0 <= s < B
            assert q0 >= (1 << 30) or q0 < count[s], what      # a live tile starts inside its request, a dead one far beyond
        meta = t.plan_meta[KEY]
        pre = mixer.prefill_launch(meta, runner.dtype, page_size)
        dec = mixer.decode_launch(meta)
        common = dict(nh=nh, nkv=nkv, hd=hd, bs=page_size, width=width, n_pages=pages, T=T)
        if tokens:
            assert dec is None and pre is not None
            live_tiles = int(sum(-(-int(c) // 64) for c in counts))
            assert int((tile_q0 < (1 << 30)).sum()) == live_tiles, what
            busy = prefill_ranges(sec, pre, wide=wide and runner.dtype == torch.bfloat16, **common)
            assert (busy > 0) == (live_tiles > 0)
            # whatever number of runs the plan can return at this bound, the workspace asked for covers it
            if pre["parts"] > 1:
                assert pre["part_o"] >= pre["n_tiles"] * 64 * nh * pre["parts"] * hd
        else:
            assert pre is None and dec is not None
            waves = 4 if hd <= 128 else 2
            decode_ranges(sec, dec, B=B, waves=waves, **common)
        runner.cache.check()


@pytest.mark.parametrize("name,raw,page_size,wide", CASES[:4], ids=[c[0] for c in CASES[:4]])
def test_eager_steps_keep_every_index_inside_its_array(name, raw, page_size, wide):
    rng = np.random.default_rng(11)
    nh, nkv, hd = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
    max_pos = raw["max_position_embeddings"]
    for trial in range(40):
        pages = int(rng.integers(8, 3 * max_pos // page_size))
        runner, cfg = runner_on_host(raw, pages, page_size, slots=8)
        mixer = runner.model.layers[0].mixer
        ids, starts, counts = [], [], []
        for i in range(int(rng.integers(1, 7))):
            count = int(rng.choice([1, 1, 2, 7, 63, 64, 65, 130, 300]))
            start = int(rng.integers(0, max(1, runner.max_position - count)))
            if start + count > runner.max_position or not runner.cache.can_extend(i, start + count):
                continue
            runner.cache.add(i)
            runner.cache.extend(i, start + count)
            runner.cache.commit(i, start)
            ids.append(i), starts.append(start), counts.append(count)
        if not ids:
            continue
        ids, starts, counts = np.asarray(ids, np.int64), np.asarray(starts, np.int32), np.asarray(counts, np.int32)
        toks = rng.integers(0, raw["vocab_size"], int(counts.sum())).astype(np.int32)
        t = runner.step_tables(ids, starts, counts, toks, (np.cumsum(counts) - 1).astype(np.int32))
        sec = sections(t)
        width = t.widths[0]
        slots = sec[("slot_mapping", 0)]
        assert ((slots >= 0) & (slots < pages * page_size)).all() and len(set(slots.tolist())) == t.T
        meta = t.plan_meta[KEY]
        common = dict(nh=nh, nkv=nkv, hd=hd, bs=page_size, width=width, n_pages=pages, T=t.T)
        pre, dec = mixer.prefill_launch(meta, runner.dtype, page_size), mixer.decode_launch(meta)
        if pre is not None:
            assert prefill_ranges(sec, pre, wide=wide, **common) > 0
        if dec is not None:
            decode_ranges(sec, dec, B=t.B, waves=4 if hd <= 128 else 2, **common)
        assert (pre is not None) == bool((counts > 1).any()) and (dec is not None) == bool((counts == 1).any())


def test_a_runner_is_built_without_a_device_and_refuses_to_launch_without_one():
    from lyapunov_engine_amd.kernels.ops import KernelError

    runner, cfg = runner_on_host(TINY_A, 16, 4)
    runner.cache.add(0)
    runner.cache.extend(0, 3)
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from lyapunov_engine_amd.engine.runner import StepEntry
    with pytest.raises(KernelError, match="no GPU"):
        runner.step([StepEntry(0, [1, 2, 3], 0, [2])])
