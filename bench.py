"""Flagship serving benchmark (driver contract).

Default ``--mode serve`` measures the BASELINE.json headline metric END TO
END: output tokens/s delivered to gRPC ``GenerateStream`` clients (+ p50
TTFT), against the real dual-front-end server on the Llama-3-8B bf16 config
with synthetic prompts / random-init weights.  The timed region is EXACTLY
``--steps`` engine steps, barrier+``torch.cuda.synchronize()``-bracketed on
both sides inside the engine process (CLOCK_MONOTONIC timestamps t0/t1
exposed via the VTA_BENCH ``/bench/window`` endpoint); the reported value is
the number of tokens the clients RECEIVED over the wire inside [t0, t1)
divided by t1-t0.  At steady state with a full always-on decode batch this
is the serving throughput of the whole stack: scheduler + HIP kernels +
sampler + detokenizer + pipe transport + proto encode + gRPC delivery.

``--mode engine`` times the bare engine step loop (scheduler + forward +
sampler + detokenizer, no wire) — the r1 bench, kept for comparison.

For ``--gpus N`` the driver launches this under torchrun, one rank per GPU
over RCCL (strong scaling: same model TP=N, same batch).  Rank 0 spawns the
server process (which becomes TP rank 0 of the group via the inherited
torchrun env) and drives the client load; ranks >0 run the broadcast worker
loop.  The window barrier spans all ranks, so rank 0's elapsed is the MAX
over ranks by construction.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=32)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--mode", choices=["serve", "engine", "arch"], default="serve",
                   help="arch: prefill/decode throughput of the Dolodra design "
                        "beside a llama of equal size (engine loop, random weights)")
    p.add_argument("--arch-sizes", type=str, default="s,m",
                   help="arch mode: comma list of sizes (s, m)")
    p.add_argument("--arch-models", type=str, default="dolodra,llama",
                   help="arch mode: which models to run (dolodra, kezunex, relerax, gumozen, "
                        "llama)")
    p.add_argument("--model", type=str, default="llama-3-8b")
    p.add_argument("--batch", type=int, default=512)
    p.add_argument("--prompt-len", type=int, default=512)
    p.add_argument("--dtype", type=str, default="bfloat16")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--top-n", type=int, default=0,
                   help="request top-N token details (logprob path) per stream")
    p.add_argument("--enforce-eager", action="store_true",
                   help="disable hipGraph decode capture (fallback-path check)")
    p.add_argument("--kv-cache-dtype", type=str, default="auto",
                   choices=["auto", "fp8"],
                   help="KV cache storage (fp8 is an ALTERNATE, non-headline "
                        "config; the BASELINE metric is bf16)")
    p.add_argument("--device", type=str, default=None)
    p.add_argument("--ttft-samples", type=int, default=5)
    p.add_argument("--grpc-port", type=int, default=18033)
    p.add_argument("--http-port", type=int, default=18080)
    p.add_argument("--timing", action="store_true",
                   help="engine mode: per-phase step timing to stderr")
    p.add_argument("--server-log", type=str, default="bench_server.log")
    return p.parse_args()


def result_json(args, *, value, ms_per_step, tp, extra_config):
    cfg = {
        "model": args.model,
        "global_batch": args.batch,
        "seq_len": args.prompt_len,
        "parallelism": f"tp{tp}",
        "decode_context": args.prompt_len,
    }
    cfg.update(extra_config)
    return {
        "metric": "grpc_stream_output_tokens_per_s"
        if args.mode == "serve" else "engine_output_tokens_per_s",
        "value": round(value, 2),
        "unit": "tokens/s",
        "n_gpus": args.gpus,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "strong",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype.startswith("b") else args.dtype,
        "data": "synthetic",
        "config": cfg,
    }


# ---------------------------------------------------------------------------
# serve mode: the BASELINE wire metric
# ---------------------------------------------------------------------------

def serve_worker_rank(args, device: str) -> None:
    """Ranks >0 under torchrun: build the TP shard, serve broadcast batches."""
    from vllm_tgis_adapter_amd.engine.worker import Worker
    from vllm_tgis_adapter_amd.parallel import init_distributed

    cfg = engine_config(args, device, tp=args.gpus)
    init_distributed(args.gpus, device=device)
    worker = Worker(cfg)
    worker.init_kv_cache()
    try:
        worker.worker_loop()
    except RuntimeError:
        # rank 0's server process exited (bench teardown) — not a failure
        pass


def engine_config(args, device: str, tp: int):
    from vllm_tgis_adapter_amd.engine import EngineConfig, ModelConfig
    from vllm_tgis_adapter_amd.engine.config import CacheConfig, SchedulerConfig

    mc = ModelConfig.from_model_arg(args.model, dtype=args.dtype)
    return EngineConfig(
        model_config=mc,
        cache_config=CacheConfig(block_size=args.block_size,
                                 kv_cache_dtype=args.kv_cache_dtype),
        scheduler_config=SchedulerConfig(
            max_num_seqs=max(args.batch, 8),
            max_num_batched_tokens=max(8192, args.batch * 2),
        ),
        device=device,
        tensor_parallel_size=tp,
        enforce_eager=args.enforce_eager,
        seed=0,
    )


async def serve_drive(args, gen_budget: int, stabilize_s: float) -> dict:
    """Client side: C always-on streams, exactly-K-steps window, TTFT probes."""
    import grpc
    import grpc.aio

    from vllm_tgis_adapter_amd.grpc import proto
    from vllm_tgis_adapter_amd.grpc.stubs import GenerationStub, HealthStub

    import asyncio
    import urllib.request

    target = f"localhost:{args.grpc_port}"

    deadline = time.time() + 600
    while True:
        try:
            async with grpc.aio.insecure_channel(target) as ch:
                resp = await HealthStub(ch).Check(
                    proto.HealthCheckRequest(service=""))
                if resp.status == 1:
                    break
        except Exception:
            pass
        if time.time() > deadline:
            raise TimeoutError("server never became healthy")
        await asyncio.sleep(2)

    channel = grpc.aio.insecure_channel(
        target, options=[("grpc.max_concurrent_streams", 4096)])
    stub = GenerationStub(channel)
    # ~prompt_len tokens with the byte-level synthetic tokenizer ("ab " = 3)
    text = "ab " * max(1, args.prompt_len // 3)

    first_token_evt = [asyncio.Event() for _ in range(args.batch)]
    # per-stream delivery log: (monotonic_ts, delta_tokens)
    deliveries: list[list] = [[] for _ in range(args.batch)]
    ttfts: list[float] = []

    async def one_stream(i: int, max_new: int, probe: bool = False):
        params = proto.Parameters()
        params.stopping.max_new_tokens = max_new
        params.stopping.min_new_tokens = max_new
        if args.top_n:
            params.response.generated_tokens = True
            params.response.token_logprobs = True
            params.response.top_n_tokens = args.top_n
        req = proto.SingleGenerationRequest(
            request=proto.GenerationRequest(text=text), params=params)
        seen = 0
        t_start = time.monotonic()
        try:
            async for msg in stub.GenerateStream(req):
                now = time.monotonic()
                if msg.generated_token_count > seen:
                    if seen == 0:
                        if probe:
                            ttfts.append((now - t_start) * 1e3)
                        else:
                            first_token_evt[i].set()
                    if not probe:
                        deliveries[i].append(
                            (now, msg.generated_token_count - seen))
                    seen = msg.generated_token_count
        except grpc.aio.AioRpcError:
            pass  # stream cancelled at teardown

    errors: list = []

    async def guarded(i):
        try:
            await one_stream(i, gen_budget)
        except Exception as e:  # surface instead of hanging the first-token wait
            errors.append(repr(e))
        finally:
            first_token_evt[i].set()

    tasks = [asyncio.get_event_loop().create_task(guarded(i))
             for i in range(args.batch)]
    await asyncio.gather(*(e.wait() for e in first_token_evt))
    if errors:
        raise RuntimeError(f"streams failed: {errors[0]} (+{len(errors)-1} more)")
    # let the delivery pipeline reach steady state: the prefill-ramp backlog
    # must drain BEFORE t0, otherwise lag shrinking across the window counts
    # pre-window production as in-window delivery (overstates the value)
    await asyncio.sleep(stabilize_s)

    # every stream is decoding: arm the exactly-K-steps window
    def _post():
        body = json.dumps({"warmup": args.warmup, "steps": args.steps}).encode()
        req = urllib.request.Request(
            f"http://localhost:{args.http_port}/bench/window", data=body,
            headers={"Content-Type": "application/json"})
        return json.loads(urllib.request.urlopen(req, timeout=600).read())

    window = await asyncio.get_event_loop().run_in_executor(None, _post)
    t0, t1 = window["t0"], window["t1"]

    # p50 TTFT probes while the batch is still decoding (loaded TTFT)
    for _ in range(args.ttft_samples):
        await one_stream(0, 2, probe=True)

    # allow in-flight deliveries to land, then stop the load
    await asyncio.sleep(0.5)
    for t in tasks:
        t.cancel()
    await asyncio.gather(*tasks, return_exceptions=True)
    await channel.close()

    wire_tokens = sum(
        d for log in deliveries for (ts, d) in log if t0 <= ts < t1)
    ttfts.sort()
    return {
        "window": window,
        "wire_tokens": wire_tokens,
        "p50_ttft_ms": ttfts[len(ttfts) // 2] if ttfts else None,
    }


def run_serve(args, device: str) -> None:
    import asyncio
    import subprocess

    rank = int(os.environ.get("RANK", "0"))
    if args.gpus > 1 and rank != 0:
        serve_worker_rank(args, device)
        return

    cmd = [
        sys.executable, "-m", "vllm_tgis_adapter_amd",
        "--model-name", args.model, "--dtype", args.dtype,
        "--device", device,
        "--max-num-seqs", str(max(args.batch, 8)),
        "--max-num-batched-tokens", str(max(8192, args.batch * 2)),
        "--block-size", str(args.block_size),
        "--kv-cache-dtype", args.kv_cache_dtype,
        "--grpc-port", str(args.grpc_port), "--port", str(args.http_port),
    ]
    if args.enforce_eager:
        cmd += ["--enforce-eager"]
    if args.gpus > 1:
        cmd += ["--num-gpus", str(args.gpus)]
    env = dict(os.environ)
    env["VTA_BENCH"] = "1"
    log = open(args.server_log, "w")
    srv = subprocess.Popen(cmd, stdout=log, stderr=log, env=env)

    # budget so no stream finishes inside ramp+stabilization+warmup+window,
    # capped by the model context (prompt + min_new must fit max_model_len)
    mc = engine_config(args, device, tp=args.gpus).model_config
    stabilize_s = 3.0 if device == "cuda" else 0.5
    room = mc.max_model_len - args.prompt_len - 8
    gen_budget = min(args.warmup + args.steps + 512, room)
    if gen_budget < args.warmup + args.steps + 8:
        raise SystemExit(
            f"context too small for the step window: room={room}")
    try:
        res = asyncio.run(serve_drive(args, gen_budget, stabilize_s))
    finally:
        srv.terminate()
        try:
            srv.wait(timeout=30)
        except subprocess.TimeoutExpired:
            srv.kill()

    win = res["window"]
    elapsed = win["elapsed_s"]
    value = res["wire_tokens"] / elapsed
    out = result_json(
        args,
        value=value,
        ms_per_step=elapsed / args.steps * 1e3,
        tp=args.gpus,
        extra_config={
            "p50_ttft_ms": round(res["p50_ttft_ms"], 2)
            if res["p50_ttft_ms"] is not None else None,
            "engine_tokens_per_s": round(win["produced"] / elapsed, 1),
            "transport": "grpc GenerateStream (loopback client)",
        },
    )
    print(json.dumps(out))


# ---------------------------------------------------------------------------
# engine mode: bare step loop (r1 bench)
# ---------------------------------------------------------------------------

def run_engine(args, device: str) -> None:
    rank = int(os.environ.get("RANK", "0"))
    tp = args.gpus

    from vllm_tgis_adapter_amd import ops
    from vllm_tgis_adapter_amd.engine import LLMEngine, SamplingParams
    from vllm_tgis_adapter_amd.parallel import init_distributed

    if device == "cuda" and not ops.has_native():
        raise RuntimeError("HIP extension _C not built — run __graft_entry__.build()")

    gen_budget = args.warmup + args.steps + 16
    cfg = engine_config(args, device, tp)

    if tp > 1:
        init_distributed(tp, device=device)
    import torch.distributed as dist

    def barrier_sync():
        if tp > 1:
            dist.barrier()
        if device == "cuda":
            torch.cuda.synchronize()

    if tp > 1 and rank != 0:
        from vllm_tgis_adapter_amd.engine.worker import Worker
        from vllm_tgis_adapter_amd.parallel import tp_broadcast_object

        worker = Worker(cfg)
        worker.init_kv_cache()
        times = []
        while True:
            cmd = tp_broadcast_object(None)
            kind = cmd[0]
            if kind == "execute":
                worker.execute_batch(cmd[1])
            elif kind == "execute_packed":
                worker.execute_batch(worker.recv_packed_batch(cmd[1]))
            elif kind == "add_lora":
                worker.add_lora(cmd[1], cmd[2])
            elif kind == "barrier":
                barrier_sync()
                times.append(time.perf_counter())
            elif kind == "elapsed":
                dev = "cuda" if device == "cuda" else "cpu"
                t = torch.tensor([times[-1] - times[-2]],
                                 dtype=torch.float64, device=dev)
                dist.all_reduce(t, op=dist.ReduceOp.MAX)
            elif kind == "stop":
                return
        return

    engine = LLMEngine(cfg)
    from vllm_tgis_adapter_amd.parallel import tp_broadcast_object

    def rank0_barrier():
        if tp > 1:
            tp_broadcast_object(("barrier",))
        barrier_sync()

    mc = cfg.model_config
    vocab = mc.vocab_size
    g = torch.Generator().manual_seed(1234)

    def synth_prompt(n):
        return torch.randint(4, vocab - 4, (n,), generator=g).tolist()

    for i in range(args.batch):
        engine.add_request(
            f"bench-{i}", None, synth_prompt(args.prompt_len),
            SamplingParams(temperature=0.0,
                           max_tokens=gen_budget + args.prompt_len),
        )

    while engine.scheduler.waiting or any(
        r.num_computed_tokens < r.num_prompt_tokens
        for r in engine.scheduler.running
    ):
        engine.step()
    for _ in range(args.warmup):
        engine.step()
    if args.timing:
        from collections import defaultdict

        engine.phase_times = defaultdict(float)

    rank0_barrier()
    t0 = time.perf_counter()
    produced = 0
    for _ in range(args.steps):
        engine.step()
        produced += len(engine.worker._sampling_items)
    rank0_barrier()
    t1 = time.perf_counter()

    elapsed = t1 - t0
    if args.timing and engine.phase_times:
        pt = dict(engine.phase_times)
        n = max(1, pt.pop("steps"))
        parts = {k: round(v / n * 1e3, 3) for k, v in pt.items()}
        print(f"[timing] per-step ms over {n} steps: {parts}", file=sys.stderr)
        engine.phase_times = None
    if tp > 1:
        dev = "cuda" if device == "cuda" else "cpu"
        t = torch.tensor([elapsed], dtype=torch.float64, device=dev)
        tp_broadcast_object(("elapsed",))
        dist.all_reduce(t, op=dist.ReduceOp.MAX)
        elapsed = float(t.item())

    tokens_per_s = produced / elapsed
    ms_per_step = elapsed / args.steps * 1e3

    # TTFT: fresh single request, time to first sampled token
    ttfts = []
    for i in range(args.ttft_samples):
        rid = f"ttft-{i}"
        engine.add_request(
            rid, None, synth_prompt(args.prompt_len),
            SamplingParams(temperature=0.0, max_tokens=2),
        )
        start = time.perf_counter()
        first = None
        while first is None:
            engine.step()
            req = engine.scheduler.get_request(rid)
            if req is None or req.num_output_tokens > 0:
                first = time.perf_counter()
        ttfts.append((first - start) * 1e3)
    ttfts.sort()
    p50_ttft_ms = ttfts[len(ttfts) // 2]

    for i in range(args.batch):
        engine.abort_request(f"bench-{i}")
    for i in range(args.ttft_samples):
        engine.abort_request(f"ttft-{i}")
    if tp > 1:
        tp_broadcast_object(("stop",))

    out = result_json(
        args, value=tokens_per_s, ms_per_step=ms_per_step, tp=tp,
        extra_config={"p50_ttft_ms": round(p50_ttft_ms, 2)},
    )
    print(json.dumps(out))


# ---------------------------------------------------------------------------
# --mode arch: the Dolodra design beside the closest existing model (llama)
# at equal width / depth / parameter count, random weights, through the same
# engine loop (scheduler + forward + sampler).  Reports prefill tokens/s (all
# prompts to their first token) and decode tokens/s (K steps of a full batch).
# ---------------------------------------------------------------------------

ARCH_SIZES = {
    # ~1B-class layers: 16 heads, latent 256 + 32 rotated, window 512
    "s": dict(width=2048, layers=8, vocab=32000, heads=16, dim=128, rot=32, vdim=128,
              rank=256, window=512, ff=8448, llama_inter=5632, llama_kv_heads=4),
    # ~8B-class layers: 32 heads, latent 512 + 64 rotated, window 1024
    "m": dict(width=4096, layers=8, vocab=32000, heads=32, dim=128, rot=64, vdim=128,
              rank=512, window=1024, ff=21504, llama_inter=14336, llama_kv_heads=8),
    # CPU dry run
    "t": dict(width=64, layers=2, vocab=512, heads=4, dim=16, rot=16, vdim=16,
              rank=32, window=24, ff=192, llama_inter=128, llama_kv_heads=2),
}


def _arch_model_configs(sz: dict, dtype: str):
    from vllm_tgis_adapter_amd.engine import ModelConfig
    from vllm_tgis_adapter_amd.engine.config import _DTYPES
    from vllm_tgis_adapter_amd.models.dolodra import model_config_from_json

    layers = []
    for i in range(sz["layers"]):
        mixer = {"heads": sz["heads"], "dim": sz["dim"], "rot_dim": sz["rot"],
                 "vdim": sz["vdim"], "kv_rank": sz["rank"],
                 "scale": (sz["dim"] + sz["rot"]) ** -0.5, "mask": {"size": sz["window"]},
                 "rot": {"base": 10000.0, "dims": sz["rot"]}}
        if i % 2 == 1:
            mixer["kv_from"] = i - 1   # every second layer borrows the latent
        layers.append({"type": "latent_attention", "mixer": mixer,
                       "mlp": {"kind": "dense", "ff": sz["ff"]}})
    hf = {"architecture": "Dolodra", "vocab": sz["vocab"], "width": sz["width"],
          "layers": layers, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
          "logit_softcap": 30.0, "embedding": {"scale": sz["width"] ** 0.5},
          "canon": {"taps": 4}, "token_side": {"dim": 32}}
    dolo = model_config_from_json("dolodra-synthetic", hf)
    dolo.dtype = _DTYPES[dtype]
    llama = ModelConfig(
        model="llama-equal", architecture="llama", vocab_size=sz["vocab"],
        hidden_size=sz["width"], intermediate_size=sz["llama_inter"],
        num_layers=sz["layers"], num_heads=sz["heads"],
        num_kv_heads=sz["llama_kv_heads"], head_dim=sz["width"] // sz["heads"],
        rope_theta=500000.0, rms_norm_eps=1e-5, max_model_len=8192,
        tie_word_embeddings=False, dtype=_DTYPES[dtype])
    return dolo, llama


# Kezunex at the same widths: eight layer runs (a looped pair of layers, then
# four more), attention 128-wide heads like the llama beside it, SSD / mLSTM /
# RG-LRU sizes in the proportions their papers use (inner size = width, state
# 128; matrix-memory heads of dim x 2 dim; recurrent width = width).
KEZUNEX_SIZES = {
    "s": dict(attn=(16, 4, 128, 128), ssd=(32, 64, 128, 1), mlstm=(8, 128, 256),
              rglru=(2048, 16), ff=5632),
    "m": dict(attn=(32, 8, 128, 128), ssd=(64, 64, 128, 1), mlstm=(8, 256, 512),
              rglru=(4096, 16), ff=14336),
    "t": dict(attn=(4, 2, 16, 16), ssd=(4, 16, 16, 1), mlstm=(2, 16, 32),
              rglru=(64, 4), ff=128),
}


def _kezunex_model_config(name: str, sz: dict, dtype: str):
    from vllm_tgis_adapter_amd.engine.config import _DTYPES
    from vllm_tgis_adapter_amd.models.kezunex import model_config_from_json

    kz = KEZUNEX_SIZES[name]
    h, g, d, dv = kz["attn"]
    sh, sv, sn, sg = kz["ssd"]
    mh, md, mv = kz["mlstm"]
    rw, rb = kz["rglru"]
    ff = {"kind": "dense", "ff": kz["ff"]}
    par = {"type": "parallel", "mlp": ff, "mixer": {
        "left": {"heads": h, "kv_heads": g, "dim": d, "vdim": dv, "scale": d ** -0.5,
                 "q_temp": {"coef": 0.1, "every": 256}},
        "right": {"heads": sh, "vdim": sv, "state": sn, "groups": sg, "conv": 4,
                  "norm_groups": 1},
        "left_scale": 0.5, "right_scale": 0.5}}
    mls = {"type": "mlstm", "mlp": None,
           "mixer": {"heads": mh, "dim": md, "vdim": mv, "gate_cap": 12.0}}
    rec = {"type": "rglru", "mlp": None, "mixer": {"width": rw, "blocks": rb, "conv": 4}}
    n = sz["layers"]
    # looped [mlstm, parallel] x 2, then rglru / parallel alternating
    layers = [mls, par] + [rec if i % 2 == 0 else par for i in range(max(n - 4, 0))]
    hf = {"architecture": "Kezunex", "vocab": sz["vocab"], "width": sz["width"],
          "layers": layers, "loop": {"start": 0, "stop": 2, "times": 2},
          "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0}}
    mc = model_config_from_json("kezunex-synthetic", hf)
    mc.dtype = _DTYPES[dtype]
    return mc


# Relerax at the same widths: eight two-norm parallel layers, latent attention
# (the latent sizes of the Dolodra config above, no window) in three of four
# layers and windowed grouped-query attention with a sink (the llama's head
# shape) in the fourth; dense squared-relu feed-forwards alternate with routed
# ones whose chosen experts add up to about the dense size.
RELERAX_SIZES = {
    "s": dict(experts=16, identity=4, top=4, expert_ff=2048),
    "m": dict(experts=16, identity=4, top=4, expert_ff=5376),
    "t": dict(experts=4, identity=2, top=2, expert_ff=96),
}


def _relerax_model_config(name: str, sz: dict, dtype: str):
    from vllm_tgis_adapter_amd.engine.config import _DTYPES
    from vllm_tgis_adapter_amd.models.relerax import model_config_from_json

    rx = RELERAX_SIZES[name]
    scaling = {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}
    latent = {"heads": sz["heads"], "dim": sz["dim"], "rot_dim": sz["rot"], "vdim": sz["vdim"],
              "kv_rank": sz["rank"], "scale": (sz["dim"] + sz["rot"]) ** -0.5,
              "rot": {"base": 10000.0, "dims": sz["rot"], "scaling": scaling}}
    hd = sz["width"] // sz["heads"]
    attn = {"heads": sz["heads"], "kv_heads": sz["llama_kv_heads"], "dim": hd, "vdim": hd,
            "scale": hd ** -0.5, "mask": {"size": sz["window"]},
            "rot": {"base": 10000.0, "dims": hd // 2, "scaling": scaling}}
    dense = {"kind": "dense", "ff": sz["ff"]}
    moe = {"kind": "moe", "expert": {"ff": rx["expert_ff"]},
           "router": {"experts": rx["experts"], "identity": rx["identity"], "top": rx["top"]}}
    layers = []
    for i in range(sz["layers"]):
        kind = "attention" if i % 4 == 2 else "latent_attention"
        layers.append({"type": kind, "mixer": attn if kind == "attention" else latent,
                       "mlp": moe if i % 2 == 1 else dense})
    hf = {"architecture": "Relerax", "vocab": sz["vocab"], "width": sz["width"],
          "layers": layers, "norm": {"eps": 1e-5}}
    mc = model_config_from_json("relerax-synthetic", hf)
    mc.dtype = _DTYPES[dtype]
    return mc


# Gumozen at the same widths: eight post-norm layers [hgrn2, latent, attention,
# latent borrowing the rows of the one before] x 2, every one followed by routed
# gated experts whose chosen ones add up to about the llama's feed-forward.
# HGRN2 heads of 128 x 128 (width / 128 heads); differential attention with
# half the llama's head counts (each head has two maps of 128) and chunks of
# 2048; latent attention with the latent of the Dolodra config and queries
# through a latent three times as wide.
GUMOZEN_SIZES = {
    "s": dict(experts=16, top=4, expert_ff=1408, chunk=2048),
    "m": dict(experts=16, top=4, expert_ff=3584, chunk=2048),
    "t": dict(experts=4, top=2, expert_ff=48, chunk=24),
}


def _gumozen_model_config(name: str, sz: dict, dtype: str):
    from vllm_tgis_adapter_amd.engine.config import _DTYPES
    from vllm_tgis_adapter_amd.models.gumozen import model_config_from_json

    gz = GUMOZEN_SIZES[name]
    hd = sz["width"] // sz["heads"]
    rec = {"heads": sz["heads"], "dim": hd, "vdim": hd}
    att = {"heads": max(sz["heads"] // 2, 1), "kv_heads": max(sz["llama_kv_heads"] // 2, 1),
           "dim": hd, "vdim": hd, "scale": hd ** -0.5, "diff": 0.3,
           "mask": {"size": gz["chunk"]},
           "rot": {"base": 10000.0, "dims": hd,
                   "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 2048}}}
    lat = {"heads": sz["heads"], "dim": sz["dim"], "vdim": sz["vdim"], "kv_rank": sz["rank"],
           "q_rank": 3 * sz["rank"], "scale": sz["dim"] ** -0.5}
    moe = {"kind": "moe", "expert": {"ff": gz["expert_ff"]},
           "router": {"experts": gz["experts"], "top": gz["top"]}}
    layers = []
    for i in range(sz["layers"]):
        kind = ("hgrn2", "latent_attention", "attention", "latent_attention")[i % 4]
        mixer = dict({"hgrn2": rec, "attention": att, "latent_attention": lat}[kind])
        if i % 4 == 3:
            mixer["kv_from"] = i - 2
        layers.append({"type": kind, "mixer": mixer, "mlp": moe})
    hf = {"architecture": "Gumozen", "vocab": sz["vocab"], "width": sz["width"],
          "layers": layers, "norm": {"eps": 1e-6}}
    mc = model_config_from_json("gumozen-synthetic", hf)
    mc.dtype = _DTYPES[dtype]
    return mc


def _arch_measure(mc, args, device: str, batch: int, prompt_len: int, steps: int,
                  warmup: int) -> dict:
    from vllm_tgis_adapter_amd.engine import EngineConfig, LLMEngine, SamplingParams
    from vllm_tgis_adapter_amd.engine.config import CacheConfig, SchedulerConfig

    bs = args.block_size
    per_seq = (prompt_len + steps + warmup + 8 + bs - 1) // bs
    cfg = EngineConfig(
        model_config=mc,
        cache_config=CacheConfig(block_size=bs, num_gpu_blocks=batch * per_seq + 16),
        scheduler_config=SchedulerConfig(max_num_seqs=batch, max_num_batched_tokens=8192,
                                         prefill_admit_batch=1),
        device=device, enforce_eager=args.enforce_eager)
    engine = LLMEngine(cfg)
    sync = torch.cuda.synchronize if device == "cuda" else (lambda: None)
    g = torch.Generator().manual_seed(0)
    res = {}
    for rnd in range(2):   # round 0 warms allocators / GEMM heuristics
        for i in range(batch):
            ids = torch.randint(4, mc.vocab_size, (prompt_len,), generator=g).tolist()
            engine.add_request(f"r{rnd}-{i}", None, ids,
                               SamplingParams(temperature=0.0, max_tokens=steps + warmup + 4,
                                              min_tokens=steps + warmup + 4))
        sync()
        t0 = time.perf_counter()
        while engine.scheduler.waiting or any(r.is_prefilling for r in engine.scheduler.running):
            engine.step()
        sync()
        t1 = time.perf_counter()
        for _ in range(warmup):
            engine.step()
        sync()
        t2 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        sync()
        t3 = time.perf_counter()
        res = {"prefill_tok_s": batch * prompt_len / (t1 - t0),
               "decode_tok_s": batch * steps / (t3 - t2),
               "decode_ms_per_step": (t3 - t2) / steps * 1e3}
        for rid in [r.request_id for r in list(engine.scheduler.running)]:
            engine.abort_request(rid)
        while engine.has_unfinished():
            engine.step()
    # the engine holds reference cycles (graphs, caches): collect them now, or
    # the next model's decode steps share the process with its leftovers
    del engine
    import gc

    gc.collect()
    if device == "cuda":
        torch.cuda.empty_cache()
    return res


def run_arch(args, device: str) -> None:
    out = []
    sizes = ["t"] if device == "cpu" else args.arch_sizes.split(",")
    for name in sizes:
        sz = ARCH_SIZES[name]
        dolo, llama = _arch_model_configs(sz, args.dtype)
        batch = min(args.batch, 256) if device == "cuda" else 4
        plen = args.prompt_len if device == "cuda" else 32
        steps = args.steps if device == "cuda" else 4
        warm = args.warmup if device == "cuda" else 1
        models = [("dolodra", dolo), ("kezunex", None), ("relerax", None), ("gumozen", None),
                  ("llama", llama)]
        for label, mc in models:
            if label not in args.arch_models.split(","):
                continue
            if label == "kezunex":
                mc = _kezunex_model_config(name, sz, args.dtype)
            if label == "relerax":
                mc = _relerax_model_config(name, sz, args.dtype)
            if label == "gumozen":
                mc = _gumozen_model_config(name, sz, args.dtype)
            r = _arch_measure(mc, args, device, batch, plen, steps, warm)
            r.update(size=name, model=label, batch=batch, prompt_len=plen)
            out.append(r)
            print(f"[arch] size={name} {label:8s} batch={batch} prompt={plen}: "
                  f"prefill {r['prefill_tok_s']:.0f} tok/s, decode {r['decode_tok_s']:.0f} tok/s "
                  f"({r['decode_ms_per_step']:.2f} ms/step)", file=sys.stderr, flush=True)
    print(json.dumps({"metric": "arch_compare_tokens_per_s", "unit": "tokens/s",
                      "dtype": args.dtype, "data": "synthetic", "steps": args.steps,
                      "warmup": args.warmup, "results": out}))


def main():
    args = parse_args()
    world = int(os.environ.get("WORLD_SIZE", str(args.gpus)))
    assert world == args.gpus or args.gpus == 1, (world, args.gpus)

    device = args.device or ("cuda" if torch.cuda.is_available() else "cpu")
    if device == "cpu":
        # CPU dry-run mode (no GPU in the dev container): tiny model
        args.model = "tiny-llama"
        args.dtype = "float32"
        args.batch = min(args.batch, 64)
        args.prompt_len = min(args.prompt_len, 64)

    if args.mode == "arch":
        run_arch(args, device)
    elif args.mode == "serve":
        run_serve(args, device)
    else:
        run_engine(args, device)


if __name__ == "__main__":
    main()
