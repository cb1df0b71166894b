"""Times one kernel of the package alone, on random data of a chosen shape.

    python -m lyapunov_engine_amd.utils.kernel_bench attn_prefill --tokens 8192
    python -m lyapunov_engine_amd.utils.kernel_bench attn_decode --batch 8 --context 8192
    python -m lyapunov_engine_amd.utils.kernel_bench linear --rows 8 --out-features 16384 --in-features 2048
    python -m lyapunov_engine_amd.utils.kernel_bench residual --rows 8 --out-features 2048 --in-features 8192
    python -m lyapunov_engine_amd.utils.kernel_bench sample --rows 8 --vocab 128256 --top-k 50 --top-p 0.9
    python -m lyapunov_engine_amd.utils.kernel_bench head --rows 8
    python -m lyapunov_engine_amd.utils.kernel_bench stream --megabytes 64
    python -m lyapunov_engine_amd.utils.kernel_bench stream --megabytes 512 --blocks 256 --row-bytes 4096
    LYAPUNOV_AMD_GEMM=own python -m lyapunov_engine_amd.utils.kernel_bench linear --rows 2048 --wide 1
    python -m lyapunov_engine_amd.utils.kernel_bench rmsnorm --rows 2048 --in-features 4100 --threads 256
    python -m lyapunov_engine_amd.utils.kernel_bench floor

Prints the time per call and what it means in TFLOP/s or TB/s.  Small enough to
run under ``rocprofv3 --pmc ...`` when a kernel's counters are wanted; the
defaults are the Llama-3.2-1B shapes that bench.py runs.
"""
from __future__ import annotations

import argparse

import torch

from ..kernels import ops


def _time(fn, repeat: int) -> float:
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(repeat):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / repeat * 1e-3


def _dtype(name: str) -> torch.dtype:
    return {"bf16": torch.bfloat16, "fp32": torch.float32}[name]


def _pools(pages: int, a) -> tuple:
    dt, dev = _dtype(a.dtype), a.device
    k = torch.randn(pages, a.kv_heads, a.page_size, a.head_dim, device=dev, dtype=dt)
    v = torch.randn(pages, a.kv_heads, a.head_dim, a.page_size, device=dev, dtype=dt)
    return k, v


def attn_prefill(a) -> None:
    """One request brings ``tokens`` new tokens and ends at ``context`` keys."""
    dt, dev = _dtype(a.dtype), a.device
    S, ctx = a.tokens, max(a.context or a.tokens, a.tokens)
    pages = -(-ctx // a.page_size)
    k, v = _pools(pages, a)
    table = torch.arange(pages, dtype=torch.int32, device=dev).view(1, pages)
    q = torch.randn(S, (a.heads + 2 * a.kv_heads) * a.head_dim, device=dev, dtype=dt)
    out = torch.empty(S, a.heads * a.head_dim, device=dev, dtype=dt)
    q_start = torch.tensor([0, S], dtype=torch.int32, device=dev)
    ctx_len = torch.tensor([ctx], dtype=torch.int32, device=dev)
    n_tiles = -(-S // 64)
    tile_seq = torch.zeros(n_tiles, dtype=torch.int32, device=dev)
    tile_q0 = (torch.arange(n_tiles, dtype=torch.int32) * 64).to(dev)
    pair = 2 * (ctx - S + 64) <= ctx
    parts = a.parts or ops.attn_prefill_plan(n_tiles, ctx, a.heads, a.kv_heads, a.head_dim, dt, a.page_size)
    work = {}
    if parts > 1:
        n = n_tiles * 64 * a.heads * parts
        work = dict(parts=parts, part_o=torch.empty(n * a.head_dim, device=dev), part_ml=torch.empty(n * 2, device=dev))

    def run():
        ops.attn_prefill(q, out, k, v, table, q_start, ctx_len, tile_seq, tile_q0, n_tiles, num_heads=a.heads,
                         num_kv_heads=a.kv_heads, head_dim=a.head_dim, pair=pair, **work)

    t = _time(run, a.repeat)
    flops = 4 * a.heads * a.head_dim * (S * (ctx - S) + S * S / 2)
    print(f"attn_prefill tokens={S} context={ctx} heads={a.heads}/{a.kv_heads}x{a.head_dim} {a.dtype}: "
          f"{t * 1e6:.1f} us  {flops / t / 1e12:.1f} TFLOP/s  (keys in {parts} run{'s' if parts > 1 else ''})")


def attn_decode(a) -> None:
    """``batch`` requests with ``context`` keys each bring one token."""
    dt, dev = _dtype(a.dtype), a.device
    B, ctx = a.batch, a.context or 8192
    per = -(-ctx // a.page_size)
    k, v = _pools(B * per, a)
    table = torch.arange(B * per, dtype=torch.int32, device=dev).view(B, per)
    q = torch.randn(B, (a.heads + 2 * a.kv_heads) * a.head_dim, device=dev, dtype=dt)
    out = torch.empty(B, a.heads * a.head_dim, device=dev, dtype=dt)
    q_start = torch.arange(B + 1, dtype=torch.int32, device=dev)
    ctx_len = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    part = ops.attn_decode_plan(B, ctx, a.heads, a.kv_heads, a.head_dim)
    max_parts = -(-ctx // part)
    part_o = torch.empty(B * a.heads * max_parts * a.head_dim, device=dev)
    part_ml = torch.empty(B * a.heads * max_parts * 2, device=dev)

    def run():
        ops.attn_decode(q, out, k, v, table, q_start, ctx_len, None, B, part_o, part_ml, max_parts, part,
                        num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.head_dim)

    t = _time(run, a.repeat)
    nbytes = 2 * B * ctx * a.kv_heads * a.head_dim * k.element_size()
    print(f"attn_decode batch={B} context={ctx} heads={a.heads}/{a.kv_heads}x{a.head_dim} {a.dtype}: "
          f"{t * 1e6:.1f} us  {nbytes / t / 1e12:.2f} TB/s of keys and values ({max_parts} partitions of {part})")


def _weights(a, rows: int, cols: int) -> list:
    """The weight matrix of a product; with --cold as many copies as it takes to exceed twice the
    memory-side cache, used in turn, so that every call finds its matrix in memory as a model step does."""
    dt, dev = _dtype(a.dtype), a.device
    one = rows * cols * (2 if dt == torch.bfloat16 else 4)
    copies = max(1, -(-(512 << 20) // one)) if a.cold else 1
    return [torch.randn(rows, cols, device=dev, dtype=dt) * 0.02 for _ in range(copies)]


def _turns(ws: list):
    state = {"i": 0}

    def next_w():
        state["i"] = (state["i"] + 1) % len(ws)
        return ws[state["i"]]

    return next_w


def linear(a) -> None:
    dt, dev = _dtype(a.dtype), a.device
    x = torch.randn(a.rows, a.in_features, device=dev, dtype=dt)
    ws = _weights(a, a.out_features, a.in_features)
    next_w = _turns(ws)
    t = _time(lambda: ops.linear(x, next_w(), may_split=a.may_split), a.repeat)
    flops = 2.0 * a.rows * a.in_features * a.out_features
    w = ws[0]
    print(f"linear rows={a.rows} {a.out_features}x{a.in_features} {a.dtype}{' cold' if a.cold else ''}: {t * 1e6:.1f} us  "
          f"{flops / t / 1e12:.1f} TFLOP/s  {w.numel() * w.element_size() / t / 1e12:.2f} TB/s of weights")


def qkv(a) -> None:
    """The fused q/k/v projection with rotation and page write (``ops.linear_rope_kv``)."""
    dt, dev = _dtype(a.dtype), a.device
    M, hd, nh, nkv = a.rows, a.head_dim, a.heads, a.kv_heads
    x = torch.randn(M, a.in_features, device=dev, dtype=dt)
    ws = _weights(a, (nh + 2 * nkv) * hd, a.in_features)
    next_w = _turns(ws)
    pages = -(-M // a.page_size) + 1
    k, v = _pools(pages, a)
    positions = torch.arange(M, dtype=torch.int32, device=dev)
    slots = torch.arange(M, dtype=torch.int32, device=dev)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    ang = torch.arange(max(M, 16), dtype=torch.float32)[:, None] * inv[None, :]
    table = torch.cat([ang.cos(), ang.sin()], dim=1).contiguous().to(dev)

    def run():
        ops.linear_rope_kv(x, next_w(), positions, table, slots, k, v, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                           page_size=a.page_size)

    t = _time(run, a.repeat)
    w = ws[0]
    print(f"qkv rows={M} {w.shape[0]}x{w.shape[1]} {a.dtype}{' cold' if a.cold else ''}: {t * 1e6:.1f} us  "
          f"{w.numel() * w.element_size() / t / 1e12:.2f} TB/s of weights")


def gate_up(a) -> None:
    """The gate/up projection with the SiLU gate (``ops.linear_swiglu``, rows interleaved 8/8)."""
    dt, dev = _dtype(a.dtype), a.device
    x = torch.randn(a.rows, a.in_features, device=dev, dtype=dt)
    ws = _weights(a, a.out_features, a.in_features)
    next_w = _turns(ws)
    t = _time(lambda: ops.linear_swiglu(x, next_w(), 8), a.repeat)
    w = ws[0]
    print(f"gate_up rows={a.rows} {w.shape[0]}x{w.shape[1]} {a.dtype}{' cold' if a.cold else ''}: {t * 1e6:.1f} us  "
          f"{w.numel() * w.element_size() / t / 1e12:.2f} TB/s of weights")


def head(a) -> None:
    """The output head's kernel: float logits of ``rows`` rows, with every workgroup's row maxima."""
    dt, dev = _dtype(a.dtype), a.device
    x = torch.randn(a.rows, a.in_features, device=dev, dtype=dt)
    w = torch.randn(a.vocab, a.in_features, device=dev, dtype=dt) * 0.02
    for blocks in ([a.blocks] if a.blocks else [256, 512, 1024, 2048]):
        ops.LM_HEAD_BLOCKS = blocks
        t = _time(lambda: ops.lm_head(x, w), a.repeat)
        print(f"head rows={a.rows} {a.vocab}x{a.in_features} {a.dtype} in {blocks} workgroups: {t * 1e6:.1f} us  "
              f"{w.numel() * w.element_size() / t / 1e12:.2f} TB/s of weights")
    t = _time(lambda: ops.linear(x, w, out_dtype=torch.float32), a.repeat)
    print(f"(the weight-streaming product, one wave per 16 rows: {t * 1e6:.1f} us)")


def residual(a) -> None:
    """The product that adds to the float residual stream and prepares the next norm."""
    dt, dev = _dtype(a.dtype), a.device
    x = torch.randn(a.rows, a.in_features, device=dev, dtype=dt)
    ws = _weights(a, a.out_features, a.in_features)
    next_w = _turns(ws)
    w = ws[0]
    h = torch.zeros(a.rows, a.out_features, device=dev)
    nw = torch.ones(a.out_features, device=dev, dtype=dt)
    if ops.linear_residual(h, ops.PendingLinear(x, w, dt), nw) is False:
        raise SystemExit("the few-rows kernel does not take this shape")
    t = _time(lambda: ops.linear_residual(h, ops.PendingLinear(x, next_w(), dt), nw), a.repeat)
    print(f"residual rows={a.rows} {a.out_features}x{a.in_features} {a.dtype}{' cold' if a.cold else ''}: {t * 1e6:.1f} us  "
          f"{w.numel() * w.element_size() / t / 1e12:.2f} TB/s of weights")


def sample(a) -> None:
    """The sampler's two kernels on ``rows`` rows of random logits (temperature 0: greedy)."""
    dev = a.device
    logits = torch.randn(a.rows, a.vocab, device=dev) * 2
    temperature = torch.full((a.rows,), a.temperature, device=dev)
    top_k = torch.full((a.rows,), a.top_k, dtype=torch.int32, device=dev)
    top_p = torch.full((a.rows,), a.top_p, device=dev)
    u = torch.full((a.rows,), 0.5, device=dev)
    out = torch.empty(a.rows, dtype=torch.int32, device=dev)
    work = ops.sample_workspace(a.rows, dev)
    t = _time(lambda: ops.sample(logits, temperature, top_k, top_p, u, out, work), a.repeat)
    print(f"sample rows={a.rows} vocab={a.vocab} temperature={a.temperature} top_k={a.top_k} top_p={a.top_p}: "
          f"{t * 1e6:.1f} us")


def stream(a) -> None:
    """A kernel that only reads: ``megabytes`` of device memory once per launch, cold (another
    buffer four times the size of the memory-side cache is read in between) and warm (the same
    buffer again and again), over a range of grid sizes.  What the weight-streaming products and
    the split attention can be held against."""
    dev = a.device
    sizes = [a.megabytes] if a.megabytes else [4, 13, 34, 67, 134, 525, 2048]
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    for mb in sizes:
        src = torch.empty(mb << 20, dtype=torch.uint8, device=dev).random_()
        for blocks in ([a.blocks] if a.blocks else [256, 512, 1024, 2048, 4096]):
            sink = torch.empty(blocks * 4, dtype=torch.int32, device=dev)
            warm = _time(lambda: ops.stream_read(src, sink, blocks), a.repeat)
            cold = []
            for _ in range(5):
                ops.stream_read(flush, torch.empty(4096 * 4, dtype=torch.int32, device=dev), 4096)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                ops.stream_read(src, sink, blocks)
                e1.record()
                torch.cuda.synchronize()
                cold.append(e0.elapsed_time(e1) * 1e-3)
            c = sorted(cold)[len(cold) // 2]
            print(f"stream {mb} MiB in {blocks} workgroups: cold {c * 1e6:.1f} us {src.numel() / c / 1e12:.2f} TB/s, "
                  f"again and again {warm * 1e6:.1f} us {src.numel() / warm / 1e12:.2f} TB/s")
            if a.row_bytes and (mb << 20) % (16 * a.row_bytes) == 0:
                for whole in (False, True):
                    rows = []
                    for _ in range(5):
                        ops.stream_read(flush, torch.empty(4096 * 4, dtype=torch.int32, device=dev), 4096)
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record()
                        ops.stream_rows(src, sink, blocks, a.row_bytes, whole)
                        e1.record()
                        torch.cuda.synchronize()
                        rows.append(e0.elapsed_time(e1) * 1e-3)
                    c = sorted(rows)[len(rows) // 2]
                    how = "8 rows a wave and 128 bytes" if whole else "16 rows a wave and 64 bytes"
                    print(f"   as rows of {a.row_bytes} bytes, {how} of each per load: cold {c * 1e6:.1f} us "
                          f"{src.numel() / c / 1e12:.2f} TB/s")


def floor(a) -> None:
    """What a kernel costs that does next to nothing: 64 launches of the reading kernel over 64 KiB,
    recorded in one graph and replayed, with 1 to 1,024 workgroups; time per launch, i.e. the cost of
    a dependent step in a recorded decode step whatever it computes."""
    dev = a.device
    src = torch.empty(64 << 10, dtype=torch.uint8, device=dev).random_()
    for blocks in ([a.blocks] if a.blocks else [1, 8, 256, 1024]):
        sink = torch.empty(blocks * 4, dtype=torch.int32, device=dev)
        ops.stream_read(src, sink, blocks)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(64):
                ops.stream_read(src, sink, blocks)
        t = _time(graph.replay, a.repeat) / 64
        print(f"floor: a kernel of {blocks} workgroups that reads 64 KiB, one of 64 in a recorded graph: {t * 1e6:.2f} us")


def rmsnorm(a) -> None:
    """The norm kernels on ``rows`` rows of ``in-features`` values; ``--threads`` sets the
    workgroup size of the two-pass kernels (rows of odd lengths) instead of the built-in rule."""
    dt, dev = _dtype(a.dtype), a.device
    h = torch.randn(a.rows, a.in_features, device=dev)
    w = torch.ones(a.in_features, device=dev, dtype=dt)
    delta = torch.randn(a.rows, a.in_features, device=dev).to(dt)
    out = torch.empty(a.rows, a.in_features, device=dev, dtype=dt)
    for threads in ([a.threads] if a.threads else [0, 64, 128, 256, 512, 1024]):
        ops.norm_threads_override(threads)
        t = _time(lambda: ops.rmsnorm(h, w, 1e-5, out, delta=delta), a.repeat)
        nbytes = a.rows * a.in_features * (8 + 2 * out.element_size())
        print(f"rmsnorm rows={a.rows} width={a.in_features} {a.dtype} threads={threads or 'rule'}: {t * 1e6:.1f} us  "
              f"{nbytes / t / 1e12:.2f} TB/s")
    ops.norm_threads_override(0)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(prog="kernel_bench", description=__doc__.splitlines()[0])
    ap.add_argument("kernel", choices=["attn_prefill", "attn_decode", "linear", "qkv", "gate_up", "residual", "sample", "stream",
                                       "rmsnorm", "head", "floor"])
    ap.add_argument("--cold", action="store_true", help="linear, qkv, gate_up, residual, head: the weights come from memory "
                    "every time (copies of the matrix in turn), not from the memory-side cache")
    ap.add_argument("--megabytes", type=int, default=0, help="stream: size of the buffer (0: a range of sizes)")
    ap.add_argument("--blocks", type=int, default=0, help="stream: workgroups (0: a range)")
    ap.add_argument("--threads", type=int, default=0, help="rmsnorm: threads per row of the two-pass kernels (0: sweep)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--repeat", type=int, default=20)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--kv-heads", type=int, default=8)
    ap.add_argument("--head-dim", type=int, default=64)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--tokens", type=int, default=2048, help="attn_prefill: new tokens of the request")
    ap.add_argument("--context", type=int, default=0, help="keys per request after the step")
    ap.add_argument("--parts", type=int, default=0, help="attn_prefill: runs of keys per tile (0: as planned)")
    ap.add_argument("--batch", type=int, default=8, help="attn_decode: requests")
    ap.add_argument("--rows", type=int, default=8, help="linear: rows of activations")
    ap.add_argument("--in-features", type=int, default=2048)
    ap.add_argument("--vocab", type=int, default=128256, help="sample: width of a row of logits")
    ap.add_argument("--temperature", type=float, default=0.8)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--out-features", type=int, default=16384)
    ap.add_argument("--may-split", action="store_true", help="linear: allow partial sums over slices of K")
    ap.add_argument("--own", action="store_true", help="products of 17 to 64 rows in this package's kernel whatever "
                    "the size of the matrix (the vendor's library otherwise takes the larger ones)")
    ap.add_argument("--row-bytes", type=int, default=0, help="stream: also read the buffer as a matrix of rows of this many bytes")
    ap.add_argument("--row-tiles", type=int, default=0, help="row tiles per workgroup of that kernel (0: its rule)")
    ap.add_argument("--wide", type=int, default=-1,
                    help="many bfloat16 rows with LYAPUNOV_AMD_GEMM=own: 0 the general tiled kernel, 1 the wide kernel (tile by rule), "
                    "2 / 3 its tiles of 128 / 256 features")
    a = ap.parse_args(argv)
    ops.require_gpu()
    if a.own:
        ops.LIBRARY_ROUNDS = 1 << 20
    if a.row_tiles:
        ops.skinny_row_tiles_override(a.row_tiles)
    if a.wide >= 0:
        lib = ops.core()
        if lib.lyp_gemm_wide(a.wide) != 0:
            raise SystemExit(lib.lyp_last_error().decode())
    torch.manual_seed(0)
    {"attn_prefill": attn_prefill, "attn_decode": attn_decode, "linear": linear, "qkv": qkv, "gate_up": gate_up, "residual": residual,
     "sample": sample, "stream": stream, "rmsnorm": rmsnorm, "head": head, "floor": floor}[a.kernel](a)


if __name__ == "__main__":
    main()
