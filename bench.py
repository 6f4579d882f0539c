#!/usr/bin/env python
"""bench.py -- Llama-3-8B GGUF Q4_K_M, 512-token prefill / 256-token greedy decode on MI355X (BASELINE.json configs[1]).

    python bench.py [--gpus N] [--steps K] [--warmup W]
    python -m torch.distributed.run --nnodes=1 --nproc-per-node N --master-addr 127.0.0.1 --master-port P bench.py --gpus N ...

A "step" is ONE decode step (one new token through embedding -> 32 blocks -> norm -> lm_head -> greedy sample) at
batch 1, replayed from a HIP graph; the timed region is exactly K steps after W warm-up steps, bracketed by
barrier + torch.cuda.synchronize(); `value` = decoded tokens/s over all ranks (max time over ranks).
Method mirrors `mistralrs bench` (mistralrs-cli/src/commands/bench.rs:52-55,253-305): synthetic prompt tokens
1000 + (start+i) % 2048, EOS disabled, greedy; prefill tok/s = prompt_len / TTFT is reported next to it.
Weights are synthetic (no network), SURVEY 8(d): N(0, 0.02^2) per tensor (seed = f(tensor index)), norm weights 1 + N(0, 0.01), quantized ON THE GPU by the
device ISQ quantizers (csrc/ext_isq.hip: bit-identical to GGML's reference quantizers) with the llama.cpp Q4_K_M tensor-type map (`--weights blocks` = random
valid block bytes, the fast variant for pure kernel timing); inputs are resident in HBM when the timed region starts.
Multi-GPU: `--gpus N` with N > 1 runs ONE model tensor-parallel over the N GPUs (one process per GPU, RCCL all-reduce after every
row-parallel projection; "scaling": "strong"); launched by torch.distributed.run, or self-spawned when WORLD_SIZE is not set.
`--model auto` = Llama-3-8B (BASELINE configs[1]) for N < 8 and Llama-3-70B, 2048 prefill (configs[3]) for N = 8; `--replicas` = N independent copies.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X spec (/opt/skills/guides/MI355X_MICROARCH.md)
MFMA_PEAK = 2.5e15  # dense bf16 FLOP/s (same guide)


def q4_k_m_types(n_layers: int):
    """llama.cpp "Q4_K_M" tensor-type map: Q4_K everywhere, Q6_K for output.weight and for
    attn_v / ffn_down in the use_more_bits layers."""
    from mistralrs_amd.gguf import GgmlDType as T

    def more_bits(i):
        return i < n_layers // 8 or i >= 7 * n_layers // 8 or (i - n_layers // 8) % 3 == 2
    out = {"token_embd.weight": T.Q4K, "output.weight": T.Q6K}
    for i in range(n_layers):
        p = f"blk.{i}."
        out[p + "attn_q.weight"] = T.Q4K
        out[p + "attn_k.weight"] = T.Q4K
        out[p + "attn_v.weight"] = T.Q6K if more_bits(i) else T.Q4K
        out[p + "attn_output.weight"] = T.Q4K
        out[p + "ffn_gate.weight"] = T.Q4K
        out[p + "ffn_up.weight"] = T.Q4K
        out[p + "ffn_down.weight"] = T.Q6K if more_bits(i) else T.Q4K
    return out


def build_model(cfg, device, seed=0, max_new_tokens=4096, tp=None, quant="q4_k_m", weights="gaussian"):
    """Synthetic model of `cfg`'s (per-rank) dims.  tp = (rank, world): the column / row-parallel shards (q / k / v / gate / up rows, o / down
    columns: distributed/layers.rs:695-975,1160-1616) get rank-specific random blocks of the SHARD's shape -- the bytes and the arithmetic of a
    real shard without materialising the unsharded 40 GB tensor on every GPU -- while the replicated tensors (embedding, norms, lm_head) use
    the same seed on every rank, so all ranks compute the same logits and sample the same token."""
    import torch
    from mistralrs_amd.llama import Llama, random_qtensor
    m = Llama(cfg, device, max_new_tokens=max_new_tokens)
    d, ff, hd = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    nq, nkv = cfg.num_heads * hd, cfg.num_kv_heads * hd
    shapes = {"attn_q": (nq, d), "attn_k": (nkv, d), "attn_v": (nkv, d), "attn_output": (d, nq),
              "ffn_gate": (ff, d), "ffn_up": (ff, d), "ffn_down": (d, ff)}
    types = q4_k_m_types(cfg.num_layers)
    g = torch.Generator(device="cpu").manual_seed(seed)
    E = cfg.num_experts
    for i, (name, t) in enumerate(types.items()):
        sharded = name not in ("token_embd.weight", "output.weight")
        n, k = shapes[name.split(".")[2]] if sharded else (cfg.vocab_size, d)
        role = name.split(".")[2] if sharded else ""
        if E and role in ("ffn_gate", "ffn_up", "ffn_down"):  # Mixtral: experts stacked along the row axis, [E * n][k] packed blocks (weight_source.rs:1835)
            name, n = name.replace(role, role + "_exps"), E * n
        tseed = seed * 1000 + i + (7919 * (tp[0] + 1) if tp and sharded else 0)
        if quant == "q8_0_isq":  # in-situ quantisation: bf16 weights -> Q8_0 blocks on the device (utils/isq.rs:323-361 does this on the host cores)
            from mistralrs_amd import isq
            from mistralrs_amd.gguf import GgmlDType
            gw = torch.Generator(device=device).manual_seed(tseed)
            m.set_tensor(name, isq.quantize((torch.randn(n, k, device=device, generator=gw) * 0.02).to(torch.bfloat16), GgmlDType.Q8_0))
        elif weights == "gaussian":  # N(0, 0.02^2) through the GGML quantizer of the tensor's type (on the device, bit-identical to GGML)
            from mistralrs_amd import isq
            gw = torch.Generator(device=device).manual_seed(tseed)
            m.set_tensor(name, isq.quantize(torch.randn(n, k, device=device, generator=gw) * 0.02, t))
        else:
            m.set_tensor(name, random_qtensor(t, n, k, device, tseed))
    for i in range(cfg.num_layers if E else 0):
        m.set_tensor(f"blk.{i}.ffn_gate_inp.weight", 0.05 * torch.randn(E, d, generator=g))  # F32 router (models/mixtral.rs:262-304)
    for i in range(cfg.num_layers):
        for nm in ("attn_norm", "ffn_norm"):
            m.set_tensor(f"blk.{i}.{nm}.weight", 1.0 + 0.01 * torch.randn(d, generator=g))
    m.set_tensor("output_norm.weight", 1.0 + 0.01 * torch.randn(d, generator=g))
    return m


def host_weights(model):
    """The model's tensors as the CPU restatement takes them (GGUF name -> (ggml type id, packed uint8 [N, row_bytes]) or f32 array)."""
    w = {}
    for name, t in model._keep.items():
        if "#" in name:  # decode-layout copies of the same tensors
            continue
        if hasattr(t, "dtype") and hasattr(t, "shape") and not hasattr(t, "data_ptr"):  # QTensor
            w[name] = (t.dtype.id, t.data.cpu().numpy().reshape(t.shape[0], -1))
        else:
            w[name] = t.cpu().numpy()
    return w


def cpu_baseline(model, cfg, prompt, positions=16):
    """Reference CPU path on the host cores, the SAME synthetic model (oracle/llama_ref.py + llama_oracle.c / cpu_path_oracle.c): the parity prompt
    (`prompt`, >= 64 tokens, in ONE pass: per-row Q8_K activations, full.rs attention) followed by `positions` greedy decode steps.
      * timing ("port"): mode "cpu_fast" (= cpu order b: one f32 term per superblock, 2 kv chunks, OpenMP rows); the timed sample is its decode steps;
      * parity material, teacher-forced on that run's tokens:
          "cpu"    order a: ggml's generic GEMV order, candle's in-order rms sum, full.rs (prompt) / single_q.rs (decode) attention
          "engine" the same arithmetic in the decode engine's documented summation orders: the HIP engine must equal it bit for bit (prompt and decode)
          "exact"  dequantized weights, NO activation quantization, f64 accumulation and glue: the model every quantized evaluation approximates
    Every mode rounds K / V to bf16 on the way into the cache (the page format).  Thread count picked by a quick calibration (cgroup quotas make nproc unreliable).
    Returns (baseline record, fed tokens, {mode: [positions + 1 logit vectors: last prompt position, then after each fed token]}, {mode: LlamaRef})."""
    import numpy as np
    from mistralrs_amd.llama import rope_tables
    from oracle import llama_ref, oracle as O
    O.build()
    w = host_weights(model)
    cos, sin = rope_tables(cfg)
    # calibrate threads on one big matvec
    tname = "blk.0.ffn_gate.weight"
    x = np.random.default_rng(0).standard_normal((1, cfg.hidden_size)).astype(np.float32)
    best = (1e9, 1)
    for thr in sorted({1, 2, 4, 8, 16, 32, 64, os.cpu_count() or 1}):
        if thr > (os.cpu_count() or 1):
            continue
        O.set_threads(thr)
        O.gemv_cpu_fast(w[tname][0], w[tname][1], w[tname][1].shape[0], cfg.hidden_size, x)
        t0 = time.perf_counter()
        for _ in range(3):
            O.gemv_cpu_fast(w[tname][0], w[tname][1], w[tname][1].shape[0], cfg.hidden_size, x)
        dt = (time.perf_counter() - t0) / 3
        if dt < best[0]:
            best = (dt, thr)
    O.set_threads(best[1])
    P = len(prompt)
    nblk = (cfg.max_context_len + 31) // 32
    kw = {"cpu_b": dict(mode="cpu_fast", n_kv_chunks=2), "cpu": dict(mode="cpu"), "exact": dict(mode="exact"),
          "engine": dict(mode="engine", attn_bpw=1 if nblk <= 64 else (nblk + 63) // 64)}
    runs = {k: llama_ref.LlamaRef(cfg, w, cos, sin, kv_dtype="bf16", **v) for k, v in kw.items()}
    f32 = lambda lg: np.asarray(lg, dtype=np.float32).copy()
    # same token rule as the GPU run; the GPU side repeats exactly this (prefill of the prompt, then token by token through the decode engine)
    t0 = time.perf_counter()
    lb = [f32(runs["cpu_b"].prefill(prompt))]
    t_prompt = time.perf_counter() - t0
    fed, t0 = [], time.perf_counter()
    for i in range(positions):
        fed.append(int(lb[-1].argmax()))
        lb.append(f32(runs["cpu_b"].step(fed[-1], P + i)))
    el = time.perf_counter() - t0
    logits = {"cpu_b": lb}
    for k in ("cpu", "engine", "exact"):
        logits[k] = [f32(runs[k].prefill(prompt))] + [f32(runs[k].step(t, P + i)) for i, t in enumerate(fed)]
    base = {"value": round(positions / el, 3), "unit": "tokens/s", "cores": best[1], "kind": "port", "oracle_pinned": False,
            "prompt_tokens_per_sec": round(P / t_prompt, 2),
            "sample": f"{positions} greedy decode tokens after a {P}-token prompt (context {P}..{P + positions - 1}), same synthetic {cfg.num_layers}-layer Q4_K_M weights, "
                      f"restatement of the candle CPU path (Q8_K activations, integer block dots, OpenMP rows, gcc -O3 -march=native); "
                      f"host reports {os.cpu_count()} logical CPUs",
            "oracle_pinned_note": "candle / ggml sources are not in /root/reference (Cargo dependency): the CPU-path arithmetic is restated from the published ggml "
                                  "algorithms and pinned on the reference's own CUDA sources compiled on the host (oracle/_ref) for the block formats, not on a candle run"}
    return base, fed, logits, runs


def dropin_rate(model, cfg, prompt, steps, device):
    """What an UNMODIFIED mistralrs-core host gets from the drop-in libraries: the literal reference launch sequence of a decode step through the
    reference ABI (launch_mmvq_gguf_quantize_q8_1_* + launch_mmvq_gguf_<t>_* per projection, rotary_embedding, reshape_and_cache, paged_attention_v1 / v2,
    add_rms_norm_*; runner mode use_fused = 0) on the same weights, replayed from a HIP graph like the engine."""
    import copy
    import torch
    from mistralrs_amd.llama import Llama
    c2 = copy.copy(cfg)
    c2.use_fused, c2.decode_engine = False, False
    m2 = Llama(c2, device, max_new_tokens=steps + 16)
    for name, t in model._keep.items():
        if "#" not in name:
            m2.set_tensor(name, t)  # the same device tensors (GGUF blocks); no decode-layout copies in this mode
    assert m2.decode_path == "reference-sequence", m2.decode_path
    last = m2.prefill(prompt, 0)
    m2.set_state([int(last.argmax())], [len(prompt)])
    m2.step_counter.zero_()
    m2.capture_decode_graph(1)
    for _ in range(4):
        m2.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        m2.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    avg_ctx = len(prompt) + 4 + steps / 2
    return steps / dt, m2.decode_bytes(1, int(avg_ctx)) * (steps / dt) / HBM_PEAK


def source_digest():
    """sha256 over the kernel / runtime sources (mistral.rs_amd/csrc/**, include/*.h), file names included: identifies the BUILD a profile was taken from.  The GPU box
    has no .git, so a commit hash cannot be compared there; the committed profiles carry this digest (scripts/make_profile_summary.py) and bench.py only quotes a
    profile whose digest equals the tree it runs from."""
    import hashlib
    here = os.path.dirname(os.path.abspath(__file__))
    h = hashlib.sha256()
    files = []
    for root, sub in ((os.path.join(here, "mistral.rs_amd", "csrc"), True), (os.path.join(here, "include"), False)):
        for dp, dn, fn in os.walk(root):
            if os.path.basename(dp) == "build":
                dn[:] = []
                continue
            files += [os.path.join(dp, f) for f in fn if f.endswith((".hip", ".cuh", ".cpp", ".h"))]
            if not sub:
                break
    for f in sorted(files):
        h.update(os.path.relpath(f, here).encode() + b"\0")
        h.update(open(f, "rb").read())
    return h.hexdigest()[:16]


def committed_profile(model_name, quant="q4_k_m"):
    """Side fields of `roofline` from the committed rocprofv3 passes of THIS build (profiles/round6_{hbm_traffic,kernel_stats}.json, scripts/profile_round.sh ->
    scripts/make_profile_summary.py): HBM bytes per launch of the dominant kernel (--pmc FETCH_SIZE x 2 per the gfx950 correction + WRITE_SIZE, separate passes) and
    its average duration INSIDE the captured decode graph (kernel trace; includes the launch boundary).  Counters cannot be read from inside the timed process.  A
    profile is only quoted when its recorded source digest equals source_digest() of the running tree: otherwise both are null."""
    here = os.path.dirname(os.path.abspath(__file__))
    out = {"traffic": None, "in_graph": None}
    if "8B" not in model_name or quant != "q4_k_m":  # the profiled workload is the Q4_K_M model; ISQ Q8_0 streams twice the bytes
        return out
    dig = source_digest()
    pick = lambda ks: next(v for name, v in ks.items() if "dec_gemv_kernel<1, 2" in name.replace("(int)", "").replace("(mrs::dec::)", ""))  # NCOLS = 1, EPI_GLU
    try:
        j = json.load(open(os.path.join(here, "profiles/round6_hbm_traffic.json")))
        if j.get("source_digest") == dig:
            k = pick(j["kernels"])
            out["traffic"] = int(k["read_bytes_per_launch"] + k["write_bytes_per_launch"])
            out["traffic_source"] = "profiles/round6_hbm_traffic.json"
        else:
            out["traffic_note"] = f"profiles/round6_hbm_traffic.json is of build {j.get('source_digest')}, this tree is {dig}: not quoted"
    except (OSError, KeyError, ValueError, StopIteration):
        pass
    try:
        j = json.load(open(os.path.join(here, "profiles/round6_kernel_stats.json")))
        if j.get("source_digest") == dig:
            kk = pick(j["kernels"])
            out["in_graph"] = {"us_per_launch": round(kk["avg_us"], 2), "source": "profiles/round6_kernel_stats.json", "source_digest": dig, "commit": j.get("commit")}
        else:
            out["in_graph_note"] = f"profiles/round6_kernel_stats.json is of build {j.get('source_digest')}, this tree is {dig}: not quoted"
    except (OSError, KeyError, ValueError, StopIteration):
        pass
    return out


def timed_run(model, cfg, prompt_len, steps, warmup, batch, sync, world, dev):
    """One benchmark pass on an already built model: TTFT of a `prompt_len` prompt (reference method: prompt_len / time-to-first-token, host read-back of
    the first token included), then the HIP graph of one decode step replayed `warmup` + `steps` times, EXACTLY `steps` of them timed between
    barrier + synchronize on both sides (max over ranks)."""
    import torch
    import torch.distributed as dist
    prompt = [(1000 + i % 2048) % cfg.vocab_size for i in range(prompt_len)]
    model.prefill(prompt, 0)  # warm-up (lazy code-object loads, workspace allocation); the timed run overwrites the same pages
    sync()
    t0 = time.perf_counter()
    last = model.prefill(prompt, 0)
    first_tok = int(last.argmax())  # device -> host read-back of the first token: end of TTFT
    ttft = time.perf_counter() - t0
    B = max(1, min(8, batch))
    for sq in range(1, B):  # the other sequences of a batched run: same prompt into their own pages (untimed)
        model.prefill(prompt, 0, seq=sq)
    # ---------------- decode: HIP graph of one step, replayed
    model.set_state([first_tok] * B, [prompt_len] * B)
    model.step_counter.zero_()
    model.capture_decode_graph(B)
    for _ in range(warmup):
        model.replay()
    sync()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        model.replay()
    ev1.record()
    sync()
    wall = time.perf_counter() - t0
    dev_s = ev0.elapsed_time(ev1) / 1e3
    tmax = torch.tensor([wall], device=dev, dtype=torch.float64)
    if world > 1:
        dist.all_reduce(tmax, op=dist.ReduceOp.MAX)
    toks = model.tokens_out[0, : warmup + steps].cpu().numpy()
    assert int(model.positions[0]) == prompt_len + warmup + steps, "decode state did not advance as expected"
    return {"prompt": prompt, "ttft": ttft, "prefill_flops": model.prefill_flops(prompt_len), "B": B, "t_all": float(tmax.item()), "dev_s": dev_s, "toks": toks,
            "first_tok": first_tok}


def parity_leg(model, cfg, a, prefill_exact):
    """The parity record of the bench line: the SAME model on the GPU and on the host cores, a `--parity-prompt` (64) token prompt prefilled in ONE pass on both
    sides followed by `--parity-positions` (16) decode steps teacher-forced on the CPU run's greedy tokens.
      (1) engine vs the engine-order restatement (oracle mode "engine"): logits of the last prompt position and of every decode position, and the K / V pages the
          prefill wrote, must be IDENTICAL; the pages a token-by-token decode of the prompt writes must equal the prefill's bit for bit;
      (2) distances: engine / cpu order a / cpu order b each against the EXACT model (dequantized weights, no activation quantization, f64), per position
          (`vs_exact`): is the engine an equally valid sample of the reference arithmetic, not merely as far from a as b is;
      (3) engine vs cpu order a and the a-vs-b calibration (as in earlier rounds), argmax agreement, free-running greedy ids."""
    import numpy as np
    import torch
    P, D = a.parity_prompt, a.parity_positions
    prompt = [(1000 + i % 2048) % cfg.vocab_size for i in range(P)]
    base, fed, cl, runs = cpu_baseline(model, cfg, prompt, positions=D)
    nb = (P + cfg.block_size - 1) // cfg.block_size

    def pages():  # K / V of positions [0, P) of sequence 0 as [P, KVH, hd] bf16 bit patterns, every layer
        ks, vs = [], []
        for kc, vc in zip(model.key_caches, model.value_caches):
            blk = model.block_tables[0, :nb].long()
            k = kc[blk].permute(0, 3, 1, 2, 4).reshape(nb * cfg.block_size, cfg.num_kv_heads, cfg.head_dim)[:P]
            v = vc[blk].permute(0, 3, 1, 2).reshape(nb * cfg.block_size, cfg.num_kv_heads, cfg.head_dim)[:P]
            ks.append(k.contiguous().view(torch.int16).cpu().numpy())
            vs.append(v.contiguous().view(torch.int16).cpu().numpy())
        return np.stack(ks), np.stack(vs)

    f32 = lambda t: t.float().cpu().numpy()
    gl = [f32(model.prefill(prompt, 0))]
    kp, vp = pages()
    for i, t in enumerate(fed):
        model.set_state([t], [P + i])
        gl.append(f32(model.forward_logits(1)[0]))
    # the same prompt token by token through the decode engine, into the same pages
    for pos, t in enumerate(prompt):
        model.set_state([t], [pos])
        ld = f32(model.forward_logits(1)[0])
    kd, vd = pages()
    from oracle import oracle as O
    ref = runs["engine"]
    ko = np.stack([O.to_bf16_bits(np.stack(ref.k[l][:P])).view(np.int16) for l in range(cfg.num_layers)])
    vo = np.stack([O.to_bf16_bits(np.stack(ref.v[l][:P])).view(np.int16) for l in range(cfg.num_layers)])
    rel = lambda x, y, r: float(np.abs(x - y).max() / np.abs(r).max())
    ex = cl["exact"]
    e_x = [rel(g, c, c) for g, c in zip(gl, ex)]
    a_x = [rel(g, c, c) for g, c in zip(cl["cpu"], ex)]
    b_x = [rel(g, c, c) for g, c in zip(cl["cpu_b"], ex)]
    e_a = [rel(g, c, c) for g, c in zip(gl, cl["cpu"])]
    e_b = [rel(g, c, ca) for g, c, ca in zip(gl, cl["cpu_b"], cl["cpu"])]
    a_b = [rel(c, d, c) for c, d in zip(cl["cpu"], cl["cpu_b"])]
    ident = [bool(np.array_equal(g, c)) for g, c in zip(gl, cl["engine"])]
    e_e = [float(np.abs(g - c).max()) for g, c in zip(gl, cl["engine"])]
    ids = lambda ls: [int(x.argmax()) for x in ls]
    ratio = [e / max(x, y, 1e-12) for e, x, y in zip(e_x, a_x, b_x)]
    flips = [{"position": P - 1 + p, "cpu_a_top2_margin_over_max_logit": float((np.sort(c)[-1] - np.sort(c)[-2]) / np.abs(c).max()), "engine_vs_cpu_a": e_a[p]}
             for p, (g, c) in enumerate(zip(gl, cl["cpu"])) if int(g.argmax()) != int(c.argmax())]
    # free-running greedy from the prefilled prompt: engine vs a free-running CPU-order-a run (continues from runs["cpu"]'s prompt cache)
    cpu_a = runs["cpu"]
    for l in range(cfg.num_layers):
        del cpu_a.k[l][P:], cpu_a.v[l][P:]
    tg = tc = int(gl[0].argmax())
    tc = int(cl["cpu"][0].argmax())
    gpu_toks, cpu_toks = [tg], [tc]
    model.prefill(prompt, 0)
    for i in range(D):
        model.set_state([tg], [P + i])
        tg = int(model.forward_logits(1)[0].argmax())
        gpu_toks.append(tg)
        if gpu_toks[:-1] == cpu_toks:  # the CPU run only has to continue while the prefixes agree
            tc = int(cpu_a.step(tc, P + i).argmax())
            cpu_toks.append(tc)
    n_cmp = len(cpu_toks)
    rnd = lambda v: [round(x, 6) for x in v]
    try:
        flip = first_flip_leg(model, cfg, runs["cpu"].w)
    except Exception as e:  # reported extra
        flip = {"error": repr(e)}
    out = {
        "greedy_match": gpu_toks[:n_cmp] == cpu_toks and n_cmp == D + 1,  # vs CPU order a (the reference's own summation orders), free-running after the shared prompt
        "greedy_match_engine_order_restatement": bool(all(ident)),  # identical logits => identical ids: the engine vs the CPU evaluation of the same arithmetic in its order
        "greedy_match_between_cpu_orders": ids(cl["cpu_b"]) == ids(cl["cpu"]),  # calibration: do two CPU summation orders pick the same ids on this model (teacher-forced)
        "parity": {
            "weights": "N(0, 0.02^2) per tensor through the GGML quantizers (device ISQ, bit-identical to GGML), Q4_K_M type map" if a.weights == "gaussian" else "random valid block bytes",
            "prompt_tokens": P, "decode_positions": D, "positions": "index 0 = last prompt position, then one per decode step",
            "prompt_arithmetic": "decode engine's (mrs_gemm_qi + per-query decode attention)" if prefill_exact else "bf16-operand MFMA (NOT the reference arithmetic)",
            "oracle_pinned": False,
            "engine_vs_engine_order_restatement": {
                "bit_identical_positions": int(sum(ident)), "of": len(ident), "max_abs_logit_diff": max(e_e), "greedy_ids_identical": ids(gl) == ids(cl["engine"]),
                "kv_pages_prefill_equal_oracle": bool(np.array_equal(kp, ko) and np.array_equal(vp, vo)),
                "kv_pages_prefill_equal_token_by_token_decode": bool(np.array_equal(kp, kd) and np.array_equal(vp, vd)),
                "prefill_logits_equal_token_by_token_decode": bool(np.array_equal(gl[0], ld)),
                "what": "oracle/cpu_path_oracle.c: the reference CPU path's arithmetic (Q8_K activations, integer block dots, candle rms_norm, single_q.rs softmax with fast_exp) in the "
                        "engine's documented f32 summation orders; LlamaRef.prefill == its own step loop"},
            "vs_exact": {"engine": rnd(e_x), "cpu_order_a": rnd(a_x), "cpu_order_b": rnd(b_x), "engine_over_max_cpu": [round(r, 3) for r in ratio],
                         "engine_within_1.05x_of_max_cpu_at_every_position": bool(max(ratio) <= 1.05),
                         "mean": {"engine": round(float(np.mean(e_x)), 6), "cpu_order_a": round(float(np.mean(a_x)), 6), "cpu_order_b": round(float(np.mean(b_x)), 6)},
                         "what": "max |logits - exact| / max |exact| per position; exact = dequantized weights, f32 activations without quantization, f64 accumulation and glue, same bf16 K / V rounding"},
            "teacher_forced_max_logit_error_over_max_logit": {"engine_vs_cpu_order_a": rnd(e_a), "engine_vs_cpu_order_b": rnd(e_b), "cpu_order_a_vs_cpu_order_b": rnd(a_b)},
            "mean": {"engine_vs_cpu_order_a": round(float(np.mean(e_a)), 6), "cpu_order_a_vs_cpu_order_b": round(float(np.mean(a_b)), 6),
                     "ratio": round(float(np.mean(e_a) / max(np.mean(a_b), 1e-12)), 3)},
            "argmax_agree_with_cpu_order_a": {"engine": int(sum(x == y for x, y in zip(ids(gl), ids(cl["cpu"])))), "cpu_order_b": int(sum(x == y for x, y in zip(ids(cl["cpu_b"]), ids(cl["cpu"])))),
                                              "of": len(gl)},
            "argmax_flips": flips[:4],
            "first_flip": flip, "first_position_vs_cpu_order_a": flip.get("first_position_vs_cpu_order_a"), "positions_before_first_flip": flip.get("positions_before_first_flip"),
            "greedy_free_running": {"tokens_compared": n_cmp, "first_difference": next((i for i, (x, y) in enumerate(zip(gpu_toks, cpu_toks)) if x != y), None)},
            "note": "cpu order a = ggml generic 8-lane GEMV order + candle in-order rms sum + full.rs (prompt) / single_q.rs (decode, 1 kv chunk) attention; b = one f32 term per "
                    "superblock + 2 kv chunks. Orders that differ ONLY in f32 summation agree to ~1e-6 until a rounding difference moves one int8 activation quant across a "
                    "rounding step, then sit at the int8 noise floor of this random-weight model (profiles/round3_parity.md); the engine's arithmetic is pinned by the bit-identical "
                    "restatement, its validity as a sample of the reference arithmetic by vs_exact."}}
    return base, out


def first_flip_leg(model, cfg, ref_w, positions=6):
    """the one parity measurement that was still inferred from 2-layer models.  On THIS (32-layer) model:
      * `first_position_vs_cpu_order_a`: a 1-token prompt -- no int8 activation quant can have moved yet between two f32 summation orders except through f32 rounding
        itself -- on the engine and on LlamaRef(mode="cpu") (the reference's own orders): max |logit difference| / max |logit|;
      * `positions_before_first_flip`: the oracle in the ENGINE's order (which the HIP engine equals bit for bit, checked above) and in CPU order a decode the same
        tokens (teacher-forced on order a's greedy ids); every linear's int8 activation quants are compared, position by position: how many positions (and, inside the
        first differing position, how many linears) pass before ONE quant differs, and how many of the quants differ there."""
    import numpy as np
    from mistralrs_amd.llama import rope_tables
    from oracle import llama_ref
    cos, sin = rope_tables(cfg)
    nblk = (cfg.max_context_len + 31) // 32
    ra = llama_ref.LlamaRef(cfg, ref_w, cos, sin, kv_dtype="bf16", mode="cpu")
    re = llama_ref.LlamaRef(cfg, ref_w, cos, sin, kv_dtype="bf16", mode="engine", attn_bpw=1 if nblk <= 64 else (nblk + 63) // 64)
    tok = 1000 % cfg.vocab_size
    g0 = model.prefill([tok], 0).float().cpu().numpy().reshape(-1)
    out = {}
    first = None
    for pos in range(positions):
        ra.trace, re.trace = [], []
        la = np.asarray(ra.step(tok, pos), dtype=np.float32)
        le = np.asarray(re.step(tok, pos), dtype=np.float32)
        if pos == 0:
            out["first_position_vs_cpu_order_a"] = float(np.abs(g0 - la).max() / np.abs(la).max())
            out["first_position_engine_equals_engine_order_restatement"] = bool(np.array_equal(g0, le))
        if first is None:
            for li, ((na, qa), (ne, qe)) in enumerate(zip(ra.trace, re.trace)):
                nd = int((qa != qe).sum())
                if nd:
                    first = {"position": pos, "linears_before_it_in_that_position": li, "of_linears_per_position": len(ra.trace), "tensor": na,
                             "quants_differing": nd, "of_quants": int(qa.size), "largest_quant_step": int(np.abs(qa.astype(np.int16) - qe.astype(np.int16)).max())}
                    break
        out.setdefault("per_position_vs_cpu_order_a", []).append(round(float(np.abs(le - la).max() / np.abs(la).max()), 9))
        tok = int(la.argmax())
    ra.trace = re.trace = None
    out["positions_before_first_flip"] = positions if first is None else first["position"]
    out["first_flip"] = first
    out["what"] = ("engine-order restatement vs CPU order a on the bench model, teacher-forced on order a's ids from a 1-token prompt; per_position = max |logit difference| "
                   "/ max |logit| (engine order vs order a); a flip = one int8 activation quant of one linear differing between the two orders")
    return out


def moe_parity_leg(dev, layers=4, P=16, D=4):
    """Parity record of the configs[4] leg: a `layers`-layer model of Mixtral-8x7B's layer shape (8 experts, top-2, hidden 4096, ffn 14336),
    N(0, 0.02^2) weights through the device ISQ quantizers, on the GPU and on the host cores:
      (1) bit-exact claims, GPU vs GPU: prefill(prompt) == decoding the prompt token by token (last-position logits and every K / V page) -- the prompt runs in the decode
          engine's arithmetic (grouped exact GEMMs over the expert-sorted routes, csrc/ext_gemm_qi.hip);
      (2) distances to the CPU restatement (oracle/llama_ref.py mode "engine"; its router / expert combination is an f64 restatement of SparseMoeBlock::forward, so this is a
          tolerance, not bit identity): last prompt position + D teacher-forced decode positions, max |dlogit| / max |logit| and arg-max agreement."""
    import gc
    import numpy as np
    import torch
    from mistralrs_amd.llama import LlamaConfig, rope_tables
    from oracle import llama_ref, oracle as O
    O.build()
    cfg = LlamaConfig.mixtral_8x7b(max_batch=1, max_context_len=64, max_position_embeddings=8192)
    cfg.num_layers = layers
    model = build_model(cfg, dev, seed=0, max_new_tokens=8, quant="q4_k_m", weights="gaussian")
    exact = bool(model.prefill_is_exact)
    prompt = [(1000 + i % 2048) % cfg.vocab_size for i in range(P)]
    nb = (P + cfg.block_size - 1) // cfg.block_size

    def pages():
        out = []
        for kc, vc in zip(model.key_caches, model.value_caches):
            blk = model.block_tables[0, :nb].long()
            out.append((kc[blk].clone().view(torch.int16), vc[blk].clone().view(torch.int16)))
        return out
    f32 = lambda t: t.float().cpu().numpy()
    lp = f32(model.prefill(prompt, 0))
    pp = pages()
    for pos, t in enumerate(prompt):
        model.set_state([t], [pos])
        ld = f32(model.forward_logits(1)[0])
    pd = pages()
    same_pages = all(bool(torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])) for a, b in zip(pp, pd))
    w = host_weights(model)
    cos, sin = rope_tables(cfg)
    O.set_threads(min(64, os.cpu_count() or 1))
    ref = llama_ref.LlamaRef(cfg, w, cos, sin, kv_dtype="bf16", mode="engine", attn_bpw=1)
    for pos, t in enumerate(prompt):
        lc = np.asarray(ref.step(t, pos), dtype=np.float32)
    rel, agree = [float(np.abs(ld - lc).max() / np.abs(lc).max())], [int(ld.argmax() == lc.argmax())]
    tok = int(lc.argmax())
    for i in range(D):
        lc = np.asarray(ref.step(tok, P + i), dtype=np.float32)
        model.set_state([tok], [P + i])
        g = f32(model.forward_logits(1)[0])
        rel.append(float(np.abs(g - lc).max() / np.abs(lc).max()))
        agree.append(int(g.argmax() == lc.argmax()))
        tok = int(lc.argmax())
    out = {"model": f"{layers} layers of Mixtral-8x7B's shape (8 experts, top-2), N(0, 0.02^2) through the device ISQ quantizers (Q4_K_M type map)", "prompt_tokens": P, "decode_positions": D,
           "prompt_arithmetic": "decode engine's (exact)" if exact else "bf16-operand MFMA",
           "prefill_logits_equal_token_by_token_decode": bool(np.array_equal(lp, ld)), "kv_pages_prefill_equal_token_by_token_decode": bool(same_pages),
           "vs_cpu_restatement_max_logit_error_over_max_logit": [round(x, 6) for x in rel], "argmax_agree_with_cpu_restatement": f"{sum(agree)} / {len(agree)}",
           "oracle_pinned": False}
    del model, ref, w
    gc.collect()
    torch.cuda.empty_cache()
    return out


def extra_config(kind, dev, steps=64, warmup=4, prompt_len=512):
    """A second BASELINE.json configuration on the same GPU, after the headline run (N = 1, default flags only): the same timed_run() on a freshly built model.
    kind: "70b" = configs[3]'s model (Llama-3-70B Q4_K_M, 2048-token prompt) on ONE GPU (40 GB of weights); "q8_0_isq" = configs[2] (Llama-3-8B, every linear quantized in situ from bf16 to Q8_0 on the GPU), "mixtral" = configs[4]'s model on ONE GPU
    (Mixtral-8x7B-shaped Q4_K_M, 26 GB: fits one MI355X; the TP = 2 form is `bench.py --model mixtral --gpus 2`)."""
    import gc
    import torch
    from mistralrs_amd.llama import LlamaConfig
    t_build = time.perf_counter()
    max_ctx = (prompt_len + warmup + steps + 2 + 63) // 64 * 64
    if kind == "70b":
        prompt_len = 2048
        max_ctx = (prompt_len + warmup + steps + 2 + 63) // 64 * 64
        cfg = LlamaConfig.llama3_70b(max_batch=1, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        model = build_model(cfg, dev, seed=0, max_new_tokens=warmup + steps + 8, quant="q4_k_m", weights="gaussian")
        name, wdesc = "Llama-3-70B GGUF Q4_K_M on ONE GPU (configs[3]'s model; its TP = 8 form is `bench.py --gpus 8`)", "N(0, 0.02^2) through the device ISQ quantizers"
    elif kind == "mixtral":
        cfg = LlamaConfig.mixtral_8x7b(max_batch=1, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        model = build_model(cfg, dev, seed=0, max_new_tokens=warmup + steps + 8, quant="q4_k_m", weights="gaussian")
        name, wdesc = "Mixtral-8x7B-shaped (8 experts, top-2) GGUF Q4_K_M, TP=1", "N(0, 0.02^2) through the device ISQ quantizers (46.7 B parameters, expert stacks quantized as [8 x 14336, 4096] tensors)"
    else:
        cfg = LlamaConfig.llama3_8b(max_batch=1, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        model = build_model(cfg, dev, seed=0, max_new_tokens=warmup + steps + 8, quant="q8_0_isq", weights="gaussian")
        name, wdesc = "Llama-3-8B ISQ Q8_0 (in situ from bf16, on the GPU), TP=1", "N(0, 0.02^2) bf16 weights quantized by the device ISQ pass"
    torch.cuda.synchronize()
    t_build = time.perf_counter() - t_build

    def sync():
        torch.cuda.synchronize()
    r = timed_run(model, cfg, prompt_len, steps, warmup, 1, sync, 1, dev)
    step_bytes = model.decode_bytes(1, int(prompt_len + warmup + steps / 2))
    out = {"workload": f"{name}, {prompt_len} prefill / {steps} decode, batch 1", "weights": wdesc, "decode_tokens_per_sec": round(steps / r["t_all"], 2),
           "ms_per_step": round(1e3 * r["t_all"] / steps, 4), "steps": steps, "warmup": warmup, "step_bytes": int(step_bytes),
           "step_roofline_frac": round(step_bytes * (steps / r["t_all"]) / HBM_PEAK, 4), "prefill_tokens_per_sec": round(prompt_len / r["ttft"], 1),
           "ttft_ms": round(1e3 * r["ttft"], 2), "prefill_arithmetic": "decode engine's (exact)" if model.prefill_is_exact else "bf16-operand MFMA",
           "decode_path": model.decode_path, "build_s": round(t_build, 1)}
    if kind == "70b" and model.prefill_is_exact:  # long prompt: also the selectable bf16-operand path
        def bf16_ttft():
            model.set_prefill_mode(0)
            model.prefill(r["prompt"], 0)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            int(model.prefill(r["prompt"], 0).argmax())
            return time.perf_counter() - t0
        tb = bf16_ttft()
        out["prefill_bf16"] = {"tokens_per_sec": round(prompt_len / tb, 1), "ttft_ms": round(1e3 * tb, 2), "frac": round(r["prefill_flops"] / tb / MFMA_PEAK, 4),
                               "gemm": "fused block dequant -> bf16 MFMA (the 137 GB bf16 shadow copy is not taken by default next to three other copies of the weights)"}
        # the MI355X-first variant of the same leg: 288 GB of HBM hold the bf16 shadow copy of the 70B model as well (GGUF 41 + decode tiles 43 + MFMA-order panels 44 +
        # shadow 137 GB): built after everything above has been recorded -- if it does not fit, the note says so and nothing else is affected
        try:
            if model.build_bf16_shadow():
                ts = bf16_ttft()
                out["prefill_bf16_shadow"] = {"tokens_per_sec": round(prompt_len / ts, 1), "ttft_ms": round(1e3 * ts, 2), "frac": round(r["prefill_flops"] / ts / MFMA_PEAK, 4),
                                              "gemm": "hipBLASLt on a bf16 shadow copy of the dense linears (137 GB), built after loading", "hbm_in_use_gb": round(torch.cuda.memory_allocated() / 2 ** 30, 1)}
        except Exception as e:  # torch.OutOfMemoryError or a library refusal
            out["prefill_bf16_shadow"] = {"failed": f"{type(e).__name__}: {str(e)[:200]}"}
        try:
            model.drop_bf16_shadow()
        except Exception:
            pass
    del model
    gc.collect()
    torch.cuda.empty_cache()
    if kind == "mixtral":
        try:
            out["parity"] = moe_parity_leg(dev)
        except Exception as e:  # reported extra
            out["parity"] = {"failed": f"{type(e).__name__}: {e}"}
    return out


HYBRID_SIZES = {
    # layer lists that resemble a small and a mid-size hybrid mixture-of-experts model: three state-space layers per attention layer
    "s": dict(width=1024, layers=8, m_heads=32, m_vdim=64, state=128, groups=4, a_heads=16, a_kv=4, dim=128, vdim=128, window=1024, keep=4, experts=32, top=4, ff=512,
              shared=1024, vocab=32000),
    "m": dict(width=2048, layers=8, m_heads=64, m_vdim=64, state=128, groups=8, a_heads=32, a_kv=8, dim=128, vdim=128, window=2048, keep=4, experts=64, top=6, ff=768,
              shared=2048, vocab=32000),
}


def hybrid_leg(a, dev):
    """`--hybrid SIZE`: prefill and decode throughput of a layer-list decoder (mistralrs_amd.hybrid: state-space + windowed-attention mixers, routed experts; bf16 weights,
    random) beside the closest model the package had before -- the Llama runner with Mixtral-style sparse layers -- at equal width, depth, expert count / size and
    vocabulary (Q4_K_M blocks: that runner serves quantized weights only).  Fractions: decode = bytes a step must read (active weights + states + pages) / 8 TB/s over
    the measured step; prefill = 2 x active parameters x tokens (+ attention) / 2.5 PFLOP/s over the measured pass."""
    import torch
    from mistralrs_amd.hybrid import (AttentionSpec, HybridCache, HybridDecoder, HybridSpec, LayerSpec, Mamba2Spec, MoeSpec, RaggedBatch, RotarySpec, synthetic_weights)
    z = HYBRID_SIZES[a.hybrid]
    W = z["width"]
    layers = []
    for i in range(z["layers"]):
        ff = MoeSpec(z["experts"], z["top"], z["ff"], z["shared"])
        if i % 4 == 3:
            mx = AttentionSpec(z["a_heads"], z["a_kv"], z["dim"], z["vdim"], z["dim"] ** -0.5, z["window"], z["keep"], RotarySpec(z["dim"] // 2, 500000.0, None))
            layers.append(LayerSpec("attention", mx, ff, f"l{i}."))
        else:
            layers.append(LayerSpec("mamba2", Mamba2Spec(z["m_heads"], z["m_vdim"], z["state"], z["groups"], 4, z["groups"]), ff, f"l{i}."))
    spec = HybridSpec(z["vocab"], W, 1e-6, layers)
    prompts = [512, 2048]
    batches = [1, 8]
    bs = 32
    max_tok = max(prompts) + a.warmup + a.steps + 64
    model = HybridDecoder(spec, dev, "bfloat16", num_blocks=max(batches) * (-(-max_tok // bs) + 1) + 2, block_size=bs, state_slots=max(batches))
    model.load_weights(synthetic_weights(spec, dev, 0))
    cache = HybridCache(model)
    e = 2

    def active_weight_bytes(rows):
        tot = e * z["vocab"] * W  # head (the embedding is one row per token)
        for ls in spec.layers:
            m = ls.mixer
            if isinstance(m, Mamba2Spec):
                tot += e * W * (2 * m.inner + 2 * m.groups * m.state + m.heads) + e * W * m.inner
            else:
                tot += e * W * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + e * W * m.heads * m.vdim
            f = ls.ff
            tot += e * 3 * W * f.ff * min(f.experts, rows * f.top) + e * 3 * W * f.shared_ff + 4 * W * (f.experts + 1)
        return tot

    def flops_per_token(ctx):
        tot = 2 * z["vocab"] * W
        for ls in spec.layers:
            m = ls.mixer
            if isinstance(m, Mamba2Spec):
                tot += 2 * W * (2 * m.inner + 2 * m.groups * m.state + m.heads) + 2 * W * m.inner + 6 * m.inner * m.state
            else:
                tot += 2 * W * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + 2 * W * m.heads * m.vdim + 2 * m.heads * (m.dim + m.vdim) * min(ctx, m.window + m.keep_first)
            tot += 2 * 3 * W * (ls.ff.ff * ls.ff.top + ls.ff.shared_ff)
        return tot

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    out = {"model": f"hybrid-{a.hybrid}", "sizes": z, "dtype": "bf16", "weights": "random, drawn on the device", "prefill": {}, "decode": {}}
    with torch.no_grad():
        for T in prompts:
            assert cache.reserve(1, T)
            b = RaggedBatch.build([cache.entry(1, [(1000 + i) % z["vocab"] for i in range(T)], 0, [T - 1])], bs, dev)
            t = timed(lambda: model.forward_batch(b), 3)
            out["prefill"][str(T)] = {"tokens_per_sec": round(T / t, 1), "ms": round(1e3 * t, 3), "mfma_frac": round(T * flops_per_token(T / 2) / t / MFMA_PEAK, 4)}
            cache.release(1)
        ctx = 512
        for nb in batches:
            for r in range(nb):
                assert cache.reserve(r + 1, ctx + a.warmup + a.steps + 2)
            pre = RaggedBatch.build([cache.entry(r + 1, [(1000 + i + r) % z["vocab"] for i in range(ctx)], 0, []) for r in range(nb)], bs, dev)
            model.forward_batch(pre)
            g = model.capture_decode(nb, -(-(ctx + a.warmup + a.steps + 2) // bs))
            pos = ctx

            def step():
                nonlocal pos
                g.replay([cache.entry(r + 1, [7 + r], pos) for r in range(nb)])
                pos += 1
            for _ in range(a.warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(a.steps):
                step()
            torch.cuda.synchronize()
            t = (time.perf_counter() - t0) / a.steps
            kv = sum(e * min(pos, l.mixer.window + l.mixer.keep_first) * l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) for l in spec.layers if isinstance(l.mixer, AttentionSpec))
            nbytes = active_weight_bytes(nb) + nb * (2 * model.state_bytes_per_slot() + kv)
            out["decode"][f"batch{nb}"] = {"tokens_per_sec": round(nb / t, 1), "ms_per_step": round(1e3 * t, 4), "step_bytes": int(nbytes),
                                           "hbm_frac": round(nbytes / t / HBM_PEAK, 4)}
            for r in range(nb):
                cache.release(r + 1)
    del model, cache
    torch.cuda.empty_cache()
    # ---- the closest earlier model at equal size
    try:
        if a.hybrid_no_llama:
            raise RuntimeError("skipped (--hybrid-no-llama)")
        from mistralrs_amd.llama import LlamaConfig
        heads = W // 128
        for T in prompts[:1] if a.hybrid_quick else prompts:
            max_ctx = (T + a.warmup + a.steps + 2 + 63) // 64 * 64
            cfg = LlamaConfig(hidden_size=W, intermediate_size=z["ff"], num_layers=z["layers"], num_heads=heads, num_kv_heads=max(1, heads // 4), vocab_size=z["vocab"],
                              max_batch=1, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx), num_experts=z["experts"], num_experts_per_tok=z["top"])
            lm = build_model(cfg, dev, seed=0, max_new_tokens=a.warmup + a.steps + 8, weights="blocks")
            r = timed_run(lm, cfg, T, a.steps, a.warmup, 1, torch.cuda.synchronize, 1, dev)
            sb = lm.decode_bytes(1, int(T + a.warmup + a.steps / 2))
            out.setdefault("llama_moe_q4_k_m_equal_size", {})[str(T)] = {
                "prefill_tokens_per_sec": round(T / r["ttft"], 1), "prefill_mfma_frac": round(r["prefill_flops"] / r["ttft"] / MFMA_PEAK, 4),
                "decode_tokens_per_sec": round(a.steps / r["t_all"], 1), "decode_hbm_frac": round(sb * (a.steps / r["t_all"]) / HBM_PEAK, 4),
                "prefill_arithmetic": "decode engine's (exact)" if lm.prefill_is_exact else "bf16-operand MFMA", "decode_path": lm.decode_path}
            del lm
            torch.cuda.empty_cache()
    except Exception as ex:  # a reported side leg
        out["llama_moe_q4_k_m_equal_size"] = {"failed": f"{type(ex).__name__}: {str(ex)[:300]}"}
    d1 = out["decode"]["batch1"]
    print(json.dumps({"metric": "hybrid_decode_tokens_per_sec", "value": d1["tokens_per_sec"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": d1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"model": out["model"], "global_batch": 1, "seq_len": 512, "parallelism": "tp1"}, "hybrid": out}), flush=True)


SOBUNEX_SIZES = {
    # layer lists that resemble a small and a mid-size decoder: every second layer reads the K / V pages of the layer before it and has routed experts, the others are dense
    "s": dict(width=1024, layers=8, heads=16, kv=4, dim=64, vdim=64, window=1024, experts=32, top=4, ff=512, shared=1024, dense_ff=4096, vocab=32000),
    "m": dict(width=2048, layers=8, heads=16, kv=4, dim=128, vdim=128, window=2048, experts=64, top=6, ff=768, shared=2048, dense_ff=8192, vocab=32000),
    "l": dict(width=4096, layers=4, heads=32, kv=8, dim=128, vdim=128, window=4096, experts=64, top=6, ff=1024, shared=2048, dense_ff=14336, vocab=32000),
}


def sobunex_leg(a, dev):
    """`--sobunex SIZE`: prefill and decode throughput of a Sobunex layer list (sigmoid attention with mixed head scores, layer norms around every sublayer, xIELU and
    clamped-GLU softmax-routed feed-forwards; bf16 weights, random) beside the closest model of the package at equal size: a Gekilix list of windowed softmax attention
    layers with sigmoid-routed experts (same width, depth, heads, head sizes, window, expert count / size, vocabulary).  Then the kernels of the two designs that do like
    work, one launch each at the model's shapes: time, and the fraction of the roofline (8 TB/s for what a kernel must read and write; the attention kernels run on the
    vector ALU in both designs, their prompt passes are priced in FLOP/s of the work done)."""
    import torch
    from mistralrs_amd.hybrid import (AttentionSpec, ClampedMoeSpec, DenseSpec, HybridCache, HybridDecoder, HybridSpec, LayerSpec, MoeSpec, RaggedBatch, RotarySpec,
                                      TalkAttentionSpec, _call, synthetic_weights)
    z = SOBUNEX_SIZES[a.sobunex]
    W, H, G, D, Dv, win = z["width"], z["heads"], z["kv"], z["dim"], z["vdim"], z["window"]
    new_layers, old_layers = [], []
    for i in range(z["layers"]):
        shared = i % 2 == 1
        new_layers.append(LayerSpec("talk_attention", TalkAttentionSpec(H, G, D, Dv, D ** -0.5, win, 0.25, 256, i - 1 if shared else None),
                                    ClampedMoeSpec(z["experts"], z["top"], z["ff"], 7.0, 2.0, z["shared"], 7.0) if shared else DenseSpec(z["dense_ff"]), f"l{i}."))
        old_layers.append(LayerSpec("attention", AttentionSpec(H, G, D, Dv, D ** -0.5, win, 0, RotarySpec(D // 2, 500000.0, None)),
                                    MoeSpec(z["experts"], z["top"], z["ff"], z["shared"]), f"l{i}."))
    specs = {"sobunex": HybridSpec(z["vocab"], W, 1e-6, new_layers, norm="layer", post_norms=True), "gekilix_attention_moe": HybridSpec(z["vocab"], W, 1e-6, old_layers)}
    prompts, batches, bs, ctx = [512, 2048], [1, 8], 32, 512
    max_tok = max(prompts) + a.warmup + a.steps + 64
    blocks_per_seq = -(-(2 * win + 64) // bs)   # the single-kernel runs below place their queries one window deep

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    out = {"sizes": z, "dtype": "bf16", "weights": "random, drawn on the device", "models": {}, "kernels": {}}
    keep = {}
    with torch.no_grad():
        for name, spec in specs.items():
            model = HybridDecoder(spec, dev, "bfloat16", num_blocks=max(batches) * max(-(-max_tok // bs) + 1, blocks_per_seq) + 2, block_size=bs, state_slots=max(batches))
            model.load_weights(synthetic_weights(spec, dev, 0))
            cache = HybridCache(model)
            r = {"prefill": {}, "decode": {}}
            for T in prompts:
                assert cache.reserve(1, T)
                b = RaggedBatch.build([cache.entry(1, [(1000 + i) % z["vocab"] for i in range(T)], 0, [T - 1])], bs, dev)
                t = timed(lambda: model.forward_batch(b), 3)
                r["prefill"][str(T)] = {"tokens_per_sec": round(T / t, 1), "ms": round(1e3 * t, 3)}
                cache.release(1)
            for nb in batches:
                for q in range(nb):
                    assert cache.reserve(q + 1, ctx + a.warmup + a.steps + 2)
                model.forward_batch(RaggedBatch.build([cache.entry(q + 1, [(1000 + i + q) % z["vocab"] for i in range(ctx)], 0, []) for q in range(nb)], bs, dev))
                g = model.capture_decode(nb, -(-(ctx + a.warmup + a.steps + 2) // bs))
                pos = ctx

                def step():
                    nonlocal pos
                    g.replay([cache.entry(q + 1, [7 + q], pos) for q in range(nb)])
                    pos += 1
                for _ in range(a.warmup):
                    step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(a.steps):
                    step()
                torch.cuda.synchronize()
                t = (time.perf_counter() - t0) / a.steps
                r["decode"][f"batch{nb}"] = {"tokens_per_sec": round(nb / t, 1), "ms_per_step": round(1e3 * t, 4)}
                del g
                for q in range(nb):
                    cache.release(q + 1)
            out["models"][name] = r
            keep[name] = model.layers[0].mixer
            del model, cache
            torch.cuda.empty_cache()
        # ---- like kernels of the two designs, one launch each
        new, old = keep["sobunex"], keep["gekilix_attention_moe"]
        m = new.m
        e = 2
        kern = out["kernels"]
        for label, nseq, p0, n in (("attention_prompt", 1, 0, 2048), ("attention_prompt_deep", 1, win, 512), ("attention_decode_batch8", 8, win + 17, 1), ("attention_decode_batch1", 1, win + 17, 1)):
            ents = [{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": list(range(1 + q * blocks_per_seq, 1 + (q + 1) * blocks_per_seq)), "want": []} for q in range(nseq)]
            if ents[-1]["blocks"][-1] >= m.num_blocks:
                continue
            b = RaggedBatch.build(ents, bs, dev)
            T = b.rows
            qn = torch.randn(T, H * D, device=dev).to(torch.bfloat16)
            gate = torch.randn(T, H, device=dev)
            o = torch.empty(T, H * Dv, dtype=torch.bfloat16, device=dev)
            for c in (new.k_cache, new.v_cache, old.k_cache, old.v_cache):
                c.normal_()
            ks = min(new.KEY_SPLITS, -(-min(win, b.max_blocks * bs) // 64)) if T <= new.SPLIT_ROWS else 0   # as the mixer does: few rows share their keys between workgroups
            scratch = torch.empty(max(ks, 1), T, H * Dv, device=dev)
            t_new = timed(lambda: _call("mrs_hyb_paged_talk_sigmoid_attn", qn, new.k_cache, new.v_cache, b.block_tables, b.tok_pos, new.talk, new.pb, new.slopes, gate, H, o, T, H, G, D,
                                        Dv, bs, b.max_blocks, win, D ** -0.5, 1, b.seg_entry, b.seg_row0, b.seg_len, b.segments, b.seg_rows, scratch if ks > 1 else None, ks), 5)
            t_old = timed(lambda: _call("mrs_hyb_paged_window_attn", qn, old.k_cache, old.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, H, G, D, Dv, bs, b.max_blocks, win, 0,
                                        D ** -0.5, 1, b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT), 5)
            pairs = sum(min(p0 + i + 1, win) for i in range(n)) * nseq               # visible (query, key) pairs
            flops = 2.0 * pairs * H * (D + Dv)
            kv_bytes = nseq * e * G * (D + Dv) * min(p0 + n, win + n - 1) + T * e * H * (D + Dv)
            kern[label] = {"rows": T, "flops": flops, "min_bytes": kv_bytes,
                           "sobunex": {"us": round(1e6 * t_new, 1), "tflops": round(flops / t_new / 1e12, 2), "hbm_frac": round(kv_bytes / t_new / HBM_PEAK, 4)},
                           "gekilix": {"us": round(1e6 * t_old, 1), "tflops": round(flops / t_old / 1e12, 2), "hbm_frac": round(kv_bytes / t_old / HBM_PEAK, 4)},
                           "time_ratio": round(t_new / t_old, 2)}
        T = 2048
        x = torch.randn(T, W, device=dev)
        wv, bv = torch.randn(W, device=dev), torch.randn(W, device=dev)
        ob, o32 = torch.empty(T, W, dtype=torch.bfloat16, device=dev), torch.empty(T, W, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_layernorm", x, W, None, wv, bv, ob, o32, None, 0, T, W, 1e-6, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_rmsnorm", x, W, wv, ob, o32, None, T, W, 1, 1e-6, 1, 1, None, 0, 0), 10)
        nb_ = T * W * (4 + 2 + 4)
        kern["norm_2048_rows"] = {"min_bytes": nb_, "sobunex_layernorm": {"us": round(1e6 * t_new, 1), "hbm_frac": round(nb_ / t_new / HBM_PEAK, 4)},
                                  "gekilix_rmsnorm": {"us": round(1e6 * t_old, 1), "hbm_frac": round(nb_ / t_old / HBM_PEAK, 4)}, "time_ratio": round(t_new / t_old, 2)}
        E, top = z["experts"], z["top"]
        wr = torch.randn(E + 1, W, device=dev)
        ids, wts, gt = torch.empty(T * top, dtype=torch.int32, device=dev), torch.empty(T * top, device=dev), torch.empty(T, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_route_softmax_topk", x, wr, T, W, E, top, 2.0, ids, wts), 10)
        t_old = timed(lambda: _call("mrs_hyb_route_sigmoid_topk", x, wr, T, W, E, top, 1, ids, wts, gt), 10)
        nb_ = T * W * 4 + E * W * 4
        kern["router_2048_rows"] = {"min_bytes": nb_, "sobunex_softmax": {"us": round(1e6 * t_new, 1), "hbm_frac": round(nb_ / t_new / HBM_PEAK, 4)},
                                    "gekilix_sigmoid": {"us": round(1e6 * t_old, 1), "hbm_frac": round(nb_ / t_old / HBM_PEAK, 4)}, "time_ratio": round(t_new / t_old, 2)}
        R, ff = T * top, z["ff"]
        gu = torch.randn(R, 2 * ff, device=dev)
        act = torch.empty(R, ff, dtype=torch.bfloat16, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_glu_clamped", gu, act, R, ff, 7.0, 1.702, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_glu_silu", gu, act, R, ff, 1), 10)
        nb_ = R * ff * (8 + 2)
        kern["glu_prompt"] = {"min_bytes": nb_, "sobunex_clamped": {"us": round(1e6 * t_new, 1), "hbm_frac": round(nb_ / t_new / HBM_PEAK, 4)},
                              "gekilix_silu": {"us": round(1e6 * t_old, 1), "hbm_frac": round(nb_ / t_old / HBM_PEAK, 4)}, "time_ratio": round(t_new / t_old, 2)}
    d1 = out["models"]["sobunex"]["decode"]["batch1"]
    print(json.dumps({"metric": "sobunex_decode_tokens_per_sec", "value": d1["tokens_per_sec"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": d1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"model": f"sobunex-{a.sobunex}", "global_batch": 1, "seq_len": 512, "parallelism": "tp1"}, "sobunex": out}), flush=True)

SETOPEL_SIZES = {
    # layer lists that resemble a small, a mid-size and a large decoder: latent attention, sink attention (every second one reads the pages of the first) and retention in turn
    "s": dict(width=1024, layers=8, heads=16, kv=4, dim=64, vdim=64, rank=256, ret_heads=8, ret_dim=64, ret_vdim=128, ff=2816, streams=4, conv=4, vocab=32000),
    "m": dict(width=2048, layers=8, heads=16, kv=4, dim=128, vdim=128, rank=512, ret_heads=8, ret_dim=128, ret_vdim=256, ff=5632, streams=4, conv=4, vocab=32000),
    "l": dict(width=4096, layers=4, heads=32, kv=8, dim=128, vdim=128, rank=512, ret_heads=16, ret_dim=128, ret_vdim=256, ff=11008, streams=4, conv=4, vocab=32000),
}


def setopel_leg(a, dev):
    """`--setopel SIZE`: prefill and decode throughput of a Setopel layer list (residual streams; latent attention, sink attention with convolved projections, retention;
    SiLU-GLU feed-forwards; bf16 weights, random) beside the closest model of the package at equal size: a list of rotary softmax attention layers (in place of the two
    attention kinds) and state-space layers (in place of retention, equal state size) with dense feed-forwards of equal weight bytes and one residual stream.  Then the
    kernels of the two designs that do like work, one launch each at the model's shapes: time and the fraction of the roofline (8 TB/s for what a kernel must read and
    write; prompt attention and the recurrences run on the f32 vector ALU in both designs and are priced in FLOP/s of the work done)."""
    import torch
    from mistralrs_amd.hybrid import (AttentionSpec, DenseSpec, GluSpec, HybridCache, HybridDecoder, HybridSpec, LatentAttentionSpec, LayerSpec, Mamba2Spec, RaggedBatch,
                                      RetentionSpec, RotarySpec, SinkAttentionSpec, _call, synthetic_weights)
    z = SETOPEL_SIZES[a.setopel]
    W, H, G, D, Dv, R = z["width"], z["heads"], z["kv"], z["dim"], z["vdim"], z["rank"]
    rh, rd, rv = z["ret_heads"], z["ret_dim"], z["ret_vdim"]
    new_layers, old_layers = [], []
    first_attn = None
    for i in range(z["layers"]):
        kind = ("latent", "attention", "retention")[i % 3]
        if kind == "latent":
            new_layers.append(LayerSpec("latent_attention", LatentAttentionSpec(H, D, Dv, R, D ** -0.5), GluSpec(z["ff"]), f"l{i}."))
        elif kind == "attention":
            src = first_attn if first_attn is not None and (i // 3) % 2 == 1 else None
            new_layers.append(LayerSpec("sink_attention", SinkAttentionSpec(H, G, D, Dv, D ** -0.5, z["conv"], 30.0, 0.25, 256, src), GluSpec(z["ff"]), f"l{i}."))
            first_attn = i if first_attn is None else first_attn
        else:
            decay = [1.0 - 2.0 ** (-5 - (7.0 * h) / max(1, rh - 1)) for h in range(rh)]
            new_layers.append(LayerSpec("retention", RetentionSpec(rh, rd, rv, decay, RotarySpec(rd, 10000.0, None, "half")), None, f"l{i}."))
        if kind == "retention":
            old_layers.append(LayerSpec("mamba2", Mamba2Spec(rh, rv, rd, rh, z["conv"], 1), None, f"l{i}."))
        else:
            old_layers.append(LayerSpec("attention", AttentionSpec(H, G, D, Dv, D ** -0.5, 0, 0, RotarySpec(D // 2, 500000.0, None)), DenseSpec(3 * z["ff"] // 2), f"l{i}."))
    specs = {"setopel": HybridSpec(z["vocab"], W, 1e-6, new_layers, embed_norm="embed.norm", residual_mult=0.5, streams=z["streams"]),
             "attention_state_space_dense": HybridSpec(z["vocab"], W, 1e-6, old_layers)}
    prompts, batches, bs, ctx = [512, 2048], [1, 8], 32, 512
    max_tok = max(prompts) + a.warmup + a.steps + 64

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    out = {"sizes": z, "dtype": "bf16", "weights": "random, drawn on the device", "models": {}, "kernels": {}}
    keep = {}
    with torch.no_grad():
        for name, spec in specs.items():
            model = HybridDecoder(spec, dev, "bfloat16", num_blocks=max(batches) * (-(-max_tok // bs) + 1) + 2, block_size=bs, state_slots=max(batches))
            model.load_weights(synthetic_weights(spec, dev, 0))
            cache = HybridCache(model)
            r = {"prefill": {}, "decode": {}}
            for T in prompts:
                assert cache.reserve(1, T)
                b = RaggedBatch.build([cache.entry(1, [(1000 + i) % z["vocab"] for i in range(T)], 0, [T - 1])], bs, dev)
                t = timed(lambda: model.forward_batch(b), 3)
                r["prefill"][str(T)] = {"tokens_per_sec": round(T / t, 1), "ms": round(1e3 * t, 3)}
                cache.release(1)
            for nb in batches:
                for q in range(nb):
                    assert cache.reserve(q + 1, ctx + a.warmup + a.steps + 2)
                model.forward_batch(RaggedBatch.build([cache.entry(q + 1, [(1000 + i + q) % z["vocab"] for i in range(ctx)], 0, []) for q in range(nb)], bs, dev))
                g = model.capture_decode(nb, -(-(ctx + a.warmup + a.steps + 2) // bs))
                pos = ctx

                def step():
                    nonlocal pos
                    g.replay([cache.entry(q + 1, [7 + q], pos) for q in range(nb)])
                    pos += 1
                for _ in range(a.warmup):
                    step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(a.steps):
                    step()
                torch.cuda.synchronize()
                t = (time.perf_counter() - t0) / a.steps
                r["decode"][f"batch{nb}"] = {"tokens_per_sec": round(nb / t, 1), "ms_per_step": round(1e3 * t, 4)}
                del g
                for q in range(nb):
                    cache.release(q + 1)
            out["models"][name] = r
            keep[name] = model
            torch.cuda.empty_cache()
        # ---- like kernels of the two designs, one launch each
        new, old = keep["setopel"], keep["attention_state_space_dense"]
        kern = out["kernels"]
        e = 2
        bps = -(-(2048 + 64) // bs)

        def pair(label, t_new, t_old, nbytes=None, flops=None, **extra):
            d = {"setopel_us": round(1e6 * t_new, 1), "other_us": round(1e6 * t_old, 1), "time_ratio": round(t_new / t_old, 2), **extra}
            if nbytes is not None:
                d.update(min_bytes=nbytes[0], other_min_bytes=nbytes[1], setopel_hbm_frac=round(nbytes[0] / t_new / HBM_PEAK, 4), other_hbm_frac=round(nbytes[1] / t_old / HBM_PEAK, 4))
            if flops is not None:
                d.update(flops=flops[0], other_flops=flops[1], setopel_tflops=round(flops[0] / t_new / 1e12, 2), other_tflops=round(flops[1] / t_old / 1e12, 2))
            kern[label] = d
        sink, latent, retn = new.layers[1].mixer, new.layers[0].mixer, new.layers[2].mixer
        oattn, ossm = old.layers[1].mixer, old.layers[2].mixer
        for c in (sink.k_cache, sink.v_cache, oattn.k_cache, oattn.v_cache, latent.c_cache):
            c.normal_()
        for label, nseq, p0, n in (("attention_prompt_2048", 1, 0, 2048), ("attention_decode_batch8_ctx2048", 8, 2047, 1), ("attention_decode_batch1_ctx2048", 1, 2047, 1)):
            ents = [{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": list(range(1 + q * bps, 1 + (q + 1) * bps)), "want": []} for q in range(nseq)]
            if ents[-1]["blocks"][-1] >= new.num_blocks:
                continue
            b = RaggedBatch.build(ents, bs, dev)
            T = b.rows
            qn = torch.randn(T, H * D, device=dev).to(torch.bfloat16)
            gate = torch.randn(T, H * Dv, device=dev)
            o = torch.empty(T, H * Dv, dtype=torch.bfloat16, device=dev)
            seg = (b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT)
            t_new = timed(lambda: _call("mrs_hyb_paged_attn_opts", qn, sink.k_cache, sink.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, H, G, D, Dv, bs, b.max_blocks, 0, 0,
                                        D ** -0.5, 1, *seg, 30.0, 1, gate, H * Dv, *new.key_splits(b, H, Dv), 0), 5)
            t_old = timed(lambda: _call("mrs_hyb_paged_window_attn", qn, oattn.k_cache, oattn.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, H, G, D, Dv, bs, b.max_blocks, 0, 0,
                                        D ** -0.5, 1, *seg), 5)
            pairs = sum(p0 + i + 1 for i in range(n)) * nseq
            fl = 2.0 * pairs * H * (D + Dv)
            kvb = nseq * e * G * (D + Dv) * (p0 + n) + T * e * H * (D + Dv)
            pair("sink_" + label, t_new, t_old, (kvb + T * H * Dv * 4, kvb), (fl, fl))
            # latent attention: single rows read the cached latent rows (one shared head of `rank` dimensions for keys and values); prompt steps gather the context's
            # blocks, expand them into keys and values and read those
            if n == 1:
                qa = torch.randn(T, H * R, device=dev).to(torch.bfloat16)
                oa = torch.empty(T, H * R, dtype=torch.bfloat16, device=dev)
                t_lat = timed(lambda: _call("mrs_hyb_paged_attn_opts", qa, latent.c_cache, latent.c_cache, b.block_tables, b.tok_seq, b.tok_pos, oa, T, H, 1, R, R, bs, b.max_blocks, 0, 0,
                                            D ** -0.5, 1, *seg, 0.0, 0, None, 0, *new.key_splits(b, H, R), 0), 3)
                pair("latent_" + label, t_lat, t_old, (nseq * e * R * (p0 + n) + T * e * H * 2 * R, kvb), (2.0 * pairs * H * 2 * R, fl))
            else:
                assert latent.expands(b)
                tables, source, nblk = b.context_blocks()

                def expanded():
                    c = torch.empty(nblk * bs, R, dtype=torch.bfloat16, device=dev)
                    _call("mrs_hyb_gather_rows", latent.c_cache, source, c, nblk, bs * R * e // 4)
                    k, v = new.linear_rounded(c, latent.w_uk), new.linear_rounded(c, latent.w_uv.view(H * Dv, R))
                    _call("mrs_hyb_paged_attn_opts", qn, k, v, tables, b.tok_seq, b.tok_pos, o, T, H, H, D, Dv, bs, b.max_blocks, 0, 0, D ** -0.5, 1, *seg, 0.0, 0, None, 0, None, 0, 1)
                t_lat = timed(expanded, 3)
                fl_lat = 2.0 * pairs * H * (D + Dv) + 2.0 * nblk * bs * R * H * (D + Dv)
                pair("latent_expanded_" + label, t_lat, t_old, (nseq * e * R * (p0 + n) + T * e * H * (D + Dv), kvb), (fl_lat, fl), launches=4)
        T = 2048
        S = z["streams"]
        x, xs, y = torch.randn(T, W, device=dev), torch.randn(T, S, W, device=dev), torch.randn(T, W, device=dev)
        wv, mix, wo, wi = torch.randn(W, device=dev), torch.randn(S, S, device=dev), torch.randn(S, device=dev), torch.randn(S, device=dev)
        ob, o32 = torch.empty(T, W, dtype=torch.bfloat16, device=dev), torch.empty(T, W, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_hyper_step", xs, y, mix, wo, wi, wv, ob, None, T, S, W, 1e-6, 1, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_rmsnorm", x, W, wv, ob, None, None, T, W, 1, 1e-6, 1, 1, None, 0, 0), 10)
        pair("streams_write_read_norm_vs_norm_2048_rows", t_new, t_old, (T * W * (8 * S + 4 + 2), T * W * (4 + 2)))
        # recurrences: 2048-token prompt and a decode step of 8 sequences
        for label, ents in (("prompt_2048", [(0, 2048, 0)]), ("decode_batch8", [(600, 1, q) for q in range(8)])):
            b = RaggedBatch.build([{"tokens": [0] * n, "pos0": p0, "slot": sl, "blocks": list(range(1, 2 + (p0 + n) // bs)), "want": []} for p0, n, sl in ents], bs, dev)
            T = b.rows
            ld = rh * rv + 2 * rh * rd + rh * rv
            u = torch.randn(T, ld, device=dev) * 0.1
            yy = torch.empty(T, rh * rv, device=dev)
            steps = torch.empty(T, rh, 2, device=dev)
            carry, dk = torch.empty(b.segments, rh, rd, rv, device=dev), torch.empty(b.segments, rh, device=dev)
            t_new = timed(lambda: _call("mrs_hyb_decay_scan", u, ld, retn.decay, retn.state, yy, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, steps, carry, dk,
                                        T, b.entries, b.segments, rh, rv, rd, rh), 5)
            ms = ossm.s
            uo = torch.randn(T, 2 * ms.inner + 2 * ms.groups * ms.state + ms.heads, device=dev) * 0.1
            xbc = torch.randn(T, ms.conv_channels, device=dev) * 0.1
            t_old = timed(lambda: _call("mrs_hyb_ssd_scan", xbc, uo, ossm.dt_bias, ossm.A_log, ossm.D, ossm.ssm_state, yy, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len,
                                        b.ent_seg0, steps, carry, dk, T, b.entries, b.segments, ms.conv_channels, uo.stride(0), ms.inner + ms.conv_channels, ms.heads, ms.vdim, ms.state,
                                        ms.groups), 5)
            fl = 4.0 * T * rh * rd * rv * (3 if T > b.entries else 1)      # state update + read-out; portions run the local pass, the carry and the output pass
            nbytes = T * 4 * (2 * rh * rv + 2 * rh * rd) + len(ents) * 8 * rh * rd * rv
            pair("recurrence_" + label, t_new, t_old, (nbytes, nbytes), (fl, fl))
        # per-head products in one launch against one dense product of equal work
        T = 2048
        qh = torch.randn(T, H * D, device=dev).to(torch.bfloat16)
        wh = torch.randn(H, R, D, device=dev).to(torch.bfloat16)
        wd = torch.randn(R, H * D, device=dev).to(torch.bfloat16)
        oh = torch.empty(T, H * R, dtype=torch.bfloat16, device=dev)
        od = torch.empty(T * H, R, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_gemm_batched", qh, wh, oh, T, R, D, H * D, D, H * R, 1, H, D, R * D, R, 1), 5)
        t_old = timed(lambda: _call("mrs_hyb_gemm", qh, wd, od, T * H, R, D, D, H * D, R, 1, 0, None, 0, 0, 0), 5)
        fl = 2.0 * T * H * R * D
        pair("per_head_products_vs_dense_product_2048_rows", t_new, t_old, None, (fl, fl))
        # projections into pages: norm + page write of the latent row / convolution of q k v against norm + rotary + page write
        b = RaggedBatch.build([{"tokens": [0] * T, "pos0": 0, "slot": 0, "blocks": list(range(1, 2 + T // bs)), "want": []}], bs, dev)
        ul = torch.randn(T, H * D + R, device=dev)
        ql = torch.empty(T, H * D, dtype=torch.bfloat16, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_latent_norm_cache", ul, H * D + R, H * D, R, latent.c_norm, b.slot_mapping, ql, latent.c_cache, 1e-6, T, 1), 10)
        nqkv = H * D + G * D + G * Dv
        uq = torch.randn(T, nqkv, device=dev)
        t_old = timed(lambda: _call("mrs_hyb_qk_norm_rope_cache", uq, nqkv, oattn.q_norm, oattn.k_norm, oattn.freq, b.tok_pos, b.slot_mapping, ql, oattn.k_cache, oattn.v_cache, T, H, G, D,
                                    Dv, D // 2, bs, 1e-6, 1), 10)
        pair("latent_norm_page_write_vs_norm_rotary_page_write", t_new, t_old, (T * (H * D + R) * (4 + 2), T * nqkv * (4 + 2)))
        us = torch.randn(T, nqkv + H * Dv, device=dev)
        t_c = timed(lambda: _call("mrs_hyb_conv_qkv_cache", us, us.stride(0), sink.bias, sink.conv_w, sink.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, b.tok_pos,
                                  b.slot_mapping, ql, sink.k_cache, sink.v_cache, T, 1, H, G, D, Dv, bs, z["conv"], 0.25, 256, 1), 10)
        pair("conv_temperature_page_write_vs_norm_rotary_page_write", t_c, t_old, (T * nqkv * (4 + 2), T * nqkv * (4 + 2)), launches=2)
        ur = torch.randn(T, 2 * rh * rv + 2 * rh * rd, device=dev)
        t_r = timed(lambda: _call("mrs_hyb_rotary_half", ur, ur.stride(0), rh * rv + rh * rd, rh * rv, rh, rd, rd, retn.freq, b.tok_pos, retn.k_mult, T), 10)
        pair("half_rotary_in_place_vs_norm_rotary_page_write", t_r, t_old, (T * 2 * rh * rd * 8, T * nqkv * (4 + 2)))
    d1 = out["models"]["setopel"]["decode"]["batch1"]
    print(json.dumps({"metric": "setopel_decode_tokens_per_sec", "value": d1["tokens_per_sec"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": d1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"model": f"setopel-{a.setopel}", "global_batch": 1, "seq_len": 512, "parallelism": "tp1"}, "setopel": out}), flush=True)


GIFOPEL_SIZES = {
    # layer lists that resemble a small, a mid-size and a large decoder: matrix memory, chunked attention beside a delta rule, and a delta rule with channel decays in turn
    "s": dict(width=1024, layers=6, heads=16, kv=4, dim=64, vdim=64, chunk=1024, d_heads=8, d_kv=8, d_dim=64, d_vdim=128, r_heads=8, r_kv=4, r_dim=64, r_vdim=64, m_heads=8, m_dim=64,
              m_vdim=128, conv=4, ff=2816, experts=32, top=4, eff=512, vocab=32000),
    "m": dict(width=2048, layers=6, heads=16, kv=4, dim=128, vdim=128, chunk=2048, d_heads=16, d_kv=16, d_dim=128, d_vdim=128, r_heads=8, r_kv=4, r_dim=128, r_vdim=128, m_heads=8,
              m_dim=128, m_vdim=256, conv=4, ff=5632, experts=64, top=6, eff=768, vocab=32000),
    "l": dict(width=4096, layers=3, heads=32, kv=8, dim=128, vdim=128, chunk=4096, d_heads=32, d_kv=32, d_dim=128, d_vdim=128, r_heads=16, r_kv=8, r_dim=128, r_vdim=128, m_heads=16,
              m_dim=128, m_vdim=256, conv=4, ff=11008, experts=64, top=6, eff=1408, vocab=32000),
}


def gifopel_leg(a, dev):
    """`--gifopel SIZE`: prefill and decode throughput of a Gifopel layer list (paired norms; matrix memory, chunked sink attention beside a delta rule, delta rule with channel
    decays; dense and routed squared-ReLU feed-forwards; bf16 weights, random) beside the closest model of the package at equal size: state-space layers of equal state size
    in place of the recurrent mixers, windowed softmax attention (window = the chunk) in place of the chunked one, sigmoid-routed GLU experts of equal weight bytes.  Then the
    kernels of the two designs that do like work, one launch each at the model's shapes: time and the fraction of the roofline (8 TB/s for what a kernel must read and
    write; prompt attention and the recurrences run on the f32 vector ALU in both designs and are priced in FLOP/s of the work done)."""
    import torch
    from mistralrs_amd.hybrid import (AttentionSpec, DeltaRuleSpec, GluSpec, HybridCache, HybridDecoder, HybridSpec, LayerSpec, Mamba2Spec, MlstmSpec, MoeSpec, ParallelSpec,
                                      RaggedBatch, RotarySpec, TopkSoftmaxMoeSpec, _call, synthetic_weights)
    z = GIFOPEL_SIZES[a.gifopel]
    W, H, G, D, Dv = z["width"], z["heads"], z["kv"], z["dim"], z["vdim"]
    new_layers, old_layers = [], []
    for i in range(z["layers"]):
        kind = ("mlstm", "parallel", "channel_delta")[i % 3]
        ff_new = GluSpec(z["ff"]) if i == 0 else TopkSoftmaxMoeSpec(z["experts"], z["top"], z["eff"])
        ff_old = GluSpec(z["ff"]) if i == 0 else MoeSpec(z["experts"], z["top"], 2 * z["eff"] // 3)
        if kind == "mlstm":
            new_layers.append(LayerSpec("mlstm", MlstmSpec(z["m_heads"], z["m_dim"], z["m_vdim"], 15.0), ff_new, f"l{i}."))
            old_layers.append(LayerSpec("mamba2", Mamba2Spec(z["m_heads"], z["m_vdim"], z["m_dim"], z["m_heads"], z["conv"], 1), ff_old, f"l{i}."))
        elif kind == "parallel":
            left = AttentionSpec(H, G, D, Dv, D ** -0.5, 0, 0, RotarySpec(D // 2, 500000.0), True, chunk=z["chunk"], head_norm=True, sink=True, head_gate=True)
            right = DeltaRuleSpec(z["r_heads"], z["r_kv"], z["r_dim"], z["r_vdim"], z["conv"], "head", "silu")
            new_layers.append(LayerSpec("parallel", ParallelSpec("attention", left, "delta_rule", right), ff_new, f"l{i}."))
            old_layers.append(LayerSpec("attention", AttentionSpec(H, G, D, Dv, D ** -0.5, z["chunk"], 0, RotarySpec(D // 2, 500000.0)), None, f"l{i}a."))
            old_layers.append(LayerSpec("mamba2", Mamba2Spec(z["r_heads"], z["r_vdim"], z["r_dim"], z["r_kv"], z["conv"], 1), ff_old, f"l{i}."))
        else:
            new_layers.append(LayerSpec("delta_rule", DeltaRuleSpec(z["d_heads"], z["d_kv"], z["d_dim"], z["d_vdim"], z["conv"], "channel", "sigmoid_lowrank"), ff_new, f"l{i}."))
            old_layers.append(LayerSpec("mamba2", Mamba2Spec(z["d_heads"], z["d_vdim"], z["d_dim"], z["d_kv"], z["conv"], 1), ff_old, f"l{i}."))
    specs = {"gifopel": HybridSpec(z["vocab"], W, 1e-6, new_layers, head="embed", norm="rms", parallel_sublayers=True),
             "state_space_window_attention_moe": HybridSpec(z["vocab"], W, 1e-6, old_layers)}
    prompts, batches, bs, ctx = [512, 2048], [1, 8], 32, 512
    max_tok = max(prompts) + a.warmup + a.steps + 64

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    out = {"sizes": z, "dtype": "bf16", "weights": "random, drawn on the device", "models": {}, "kernels": {}}
    keep = {}
    with torch.no_grad():
        for name, spec in specs.items():
            model = HybridDecoder(spec, dev, "bfloat16", num_blocks=max(batches) * (-(-max_tok // bs) + 1) + 2, block_size=bs, state_slots=max(batches))
            model.load_weights(synthetic_weights(spec, dev, 0))
            cache = HybridCache(model)
            r = {"prefill": {}, "decode": {}}
            for T in prompts:
                assert cache.reserve(1, T)
                b = RaggedBatch.build([cache.entry(1, [(1000 + i) % z["vocab"] for i in range(T)], 0, [T - 1])], bs, dev)
                t = timed(lambda: model.forward_batch(b), 3)
                r["prefill"][str(T)] = {"tokens_per_sec": round(T / t, 1), "ms": round(1e3 * t, 3)}
                cache.release(1)
            for nb in batches:
                for q in range(nb):
                    assert cache.reserve(q + 1, ctx + a.warmup + a.steps + 2)
                model.forward_batch(RaggedBatch.build([cache.entry(q + 1, [(1000 + i + q) % z["vocab"] for i in range(ctx)], 0, []) for q in range(nb)], bs, dev))
                g = model.capture_decode(nb, -(-(ctx + a.warmup + a.steps + 2) // bs))
                pos = ctx

                def step():
                    nonlocal pos
                    g.replay([cache.entry(q + 1, [7 + q], pos) for q in range(nb)])
                    pos += 1
                for _ in range(a.warmup):
                    step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(a.steps):
                    step()
                torch.cuda.synchronize()
                t = (time.perf_counter() - t0) / a.steps
                r["decode"][f"batch{nb}"] = {"tokens_per_sec": round(nb / t, 1), "ms_per_step": round(1e3 * t, 4)}
                del g
                for q in range(nb):
                    cache.release(q + 1)
            out["models"][name] = r
            keep[name] = model
            torch.cuda.empty_cache()
        # ---- like kernels of the two designs, one launch each
        new, old = keep["gifopel"], keep["state_space_window_attention_moe"]
        kern = out["kernels"]
        e = 2
        f32 = dict(dtype=torch.float32, device=dev)

        def pair(label, t_new, t_old, nbytes=None, flops=None, **extra):
            d = {"gifopel_us": round(1e6 * t_new, 1), "other_us": round(1e6 * t_old, 1), "time_ratio": round(t_new / t_old, 2), **extra}
            if nbytes is not None:
                d.update(min_bytes=nbytes[0], other_min_bytes=nbytes[1], gifopel_hbm_frac=round(nbytes[0] / t_new / HBM_PEAK, 4), other_hbm_frac=round(nbytes[1] / t_old / HBM_PEAK, 4))
            if flops is not None:
                d.update(flops=flops[0], other_flops=flops[1], gifopel_tflops=round(flops[0] / t_new / 1e12, 2), other_tflops=round(flops[1] / t_old / 1e12, 2))
            kern[label] = d
        mem, both, cdel = new.layers[0].mixer, new.layers[1].mixer, new.layers[2].mixer
        ossm_m, oattn, ossm_r, ossm_d = old.layers[0].mixer, old.layers[1].mixer, old.layers[2].mixer, old.layers[3].mixer

        def ssd(b, m2):
            ms = m2.s
            T = b.rows
            uo = torch.randn(T, 2 * ms.inner + 2 * ms.groups * ms.state + ms.heads, **f32) * 0.1
            xbc = torch.randn(T, ms.conv_channels, **f32) * 0.1
            yy, steps = torch.empty(T, ms.inner, **f32), torch.empty(T, ms.heads, 2, **f32)
            carry, dk = torch.empty(b.segments, ms.heads, ms.state, ms.vdim, **f32), torch.empty(b.segments, ms.heads, **f32)
            return lambda: _call("mrs_hyb_ssd_scan", xbc, uo, m2.dt_bias, m2.A_log, m2.D, m2.ssm_state, yy, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0,
                                 steps, carry, dk, T, b.entries, b.segments, ms.conv_channels, uo.stride(0), ms.inner + ms.conv_channels, ms.heads, ms.vdim, ms.state, ms.groups)
        for label, ents in (("prompt_2048", [(0, 2048, 0)]), ("prompt_8x256", [(0, 256, q) for q in range(8)]), ("decode_batch8", [(600, 1, q) for q in range(8)]),
                            ("decode_batch1", [(600, 1, 0)])):
            b = RaggedBatch.build([{"tokens": [0] * n, "pos0": p0, "slot": sl, "blocks": list(range(1, 2 + (p0 + n) // bs)), "want": []} for p0, n, sl in ents], bs, dev)
            T = b.rows
            portion = T > b.entries
            # delta rule, a decay per key channel / per head
            for tag, mx, o2 in (("channel", cdel, ossm_d), ("head", both.right, ossm_r)):
                sp = mx.s
                c = torch.randn(T, mx.channels, **f32) * 0.1
                beta, dec, yy = torch.rand(T, sp.heads, **f32), 1 - 0.1 * torch.rand(T, sp.heads * mx.per, **f32), torch.empty(T, mx.nv, **f32)
                table, nseg, cy, tr = b.entry_table(), b.entries, None, None
                if b.seg_rows > 1 and b.entries * sp.heads * -(-sp.vdim // 16) < mx.CHAIN_WAVES:   # the mixer's own choice: segments side by side, or one chain per entry
                    *cut, n = b.segment_table(mx.SEGMENT)
                    if n > b.entries:
                        table, nseg = cut, n
                        cy, tr = torch.empty(nseg, sp.heads, sp.dim, sp.vdim, **f32), torch.empty(nseg, sp.heads, sp.dim, sp.dim, **f32)
                t_new = timed(lambda: _call("mrs_hyb_delta_scan", c, mx.channels, beta, dec, mx.state, yy, b.seq_pos0, b.seq_slot, *table, cy, tr, T, b.entries, nseg, sp.heads,
                                            sp.kv_heads, sp.dim, sp.vdim, mx.per, mx.LANES), 5)
                t_old = timed(ssd(b, o2), 5)
                st = sp.heads * sp.dim * sp.vdim
                nbytes = T * 4 * (mx.channels + mx.nv + sp.heads * (1 + mx.per)) + len(ents) * 8 * st
                pair(f"delta_{tag}_decay_{label}", t_new, t_old, (nbytes, T * 4 * (o2.s.conv_channels + o2.s.inner) + len(ents) * 8 * st),
                     (7.0 * T * st, 4.0 * T * st * (3 if portion and b.segments > b.entries else 1)))
            # matrix memory: gates + scan with the normaliser column + normaliser / head norm / gate
            sp = mem.s
            nv, nk = sp.heads * sp.vdim, sp.heads * sp.dim
            u = torch.randn(T, 2 * nv + 2 * nk + 2 * sp.heads, **f32) * 0.1
            steps, mbuf, mexp = torch.empty(T, sp.heads, 2, **f32), torch.empty(T + b.entries, sp.heads, **f32), torch.empty(T, sp.heads, **f32)
            yy = torch.empty(T, sp.heads * (sp.vdim + 1), **f32)
            carry, dk = torch.empty(b.segments, sp.heads, sp.dim, sp.vdim + 1, **f32), torch.empty(b.segments, sp.heads, **f32)
            t_g = timed(lambda: _call("mrs_hyb_exp_gates", u, u.stride(0), mem.i_col, mem.f_col, mem.bi, mem.bf, 15.0, mem.m_state, steps, mbuf, mexp, b.tok_seq, b.seq_start,
                                      b.seq_pos0, b.seq_slot, T, b.entries, sp.heads), 5)
            t_s = timed(lambda: _call("mrs_hyb_gated_scan", u, u.stride(0), steps, mem.state, yy, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, carry, dk, T,
                                      b.entries, b.segments, sp.heads, sp.vdim, sp.dim, sp.heads, 1, mem.q_mult), 5)
            t_old = timed(ssd(b, ossm_m), 5)
            st = sp.heads * sp.dim * sp.vdim
            fl = 4.0 * T * st * (3 if b.segments > b.entries else 1)
            pair(f"matrix_memory_gates_and_scan_{label}", t_g + t_s, t_old, None, (fl, fl), gates_us=round(1e6 * t_g, 1), scan_us=round(1e6 * t_s, 1))
        # attention: 2048-token prompt inside one chunk / window, decode
        bps = -(-(2048 + 64) // bs)
        att = both.left
        for c_ in (att.k_cache, att.v_cache, oattn.k_cache, oattn.v_cache):
            c_.normal_()
        for label, nseq, p0, n in (("attention_prompt_2048", 1, 0, 2048), ("attention_decode_batch8_ctx2048", 8, 2047, 1), ("attention_decode_batch1_ctx2048", 1, 2047, 1)):
            ents = [{"tokens": [0] * n, "pos0": p0, "slot": 0, "blocks": list(range(1 + q * bps, 1 + (q + 1) * bps)), "want": []} for q in range(nseq)]
            if ents[-1]["blocks"][-1] >= new.num_blocks:
                continue
            b = RaggedBatch.build(ents, bs, dev)
            T = b.rows
            qn = torch.randn(T, H * D, device=dev).to(torch.bfloat16)
            gate = torch.randn(T, H, **f32)
            o = torch.empty(T, H * Dv, dtype=torch.bfloat16, device=dev)
            seg = (b.seg_entry, b.seg_row0, b.seg_len, b.segments, RaggedBatch.SEGMENT)
            ch = max(z["chunk"], 2048)
            t_new = timed(lambda: _call("mrs_hyb_paged_attn_chunked", qn, att.k_cache, att.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, H, G, D, Dv, bs, b.max_blocks, ch,
                                        D ** -0.5, 1, *seg, 0.0, 1, att.sink, gate, H, 1, *new.key_splits(b, H, Dv, ch)), 5)
            t_old = timed(lambda: _call("mrs_hyb_paged_window_attn", qn, oattn.k_cache, oattn.v_cache, b.block_tables, b.tok_seq, b.tok_pos, o, T, H, G, D, Dv, bs, b.max_blocks, ch, 0,
                                        D ** -0.5, 1, *seg), 5)
            pairs = sum(p0 + i + 1 for i in range(n)) * nseq
            fl = 2.0 * pairs * H * (D + Dv)
            kvb = nseq * e * G * (D + Dv) * (p0 + n) + T * e * H * (D + Dv)
            pair("chunked_sink_" + label, t_new, t_old, (kvb, kvb), (fl, fl))
        # row-wise kernels at 2048 rows
        T = 2048
        b = RaggedBatch.build([{"tokens": [0] * T, "pos0": 0, "slot": 0, "blocks": list(range(1, 2 + T // bs)), "want": []}], bs, dev)
        x, wv, wv2 = torch.randn(T, W, **f32), torch.randn(W, **f32), torch.randn(W, **f32)
        ob, ob2, o32 = torch.empty(T, W, dtype=torch.bfloat16, device=dev), torch.empty(T, W, dtype=torch.bfloat16, device=dev), torch.empty(T, W, **f32)
        t_new = timed(lambda: _call("mrs_hyb_rmsnorm_pair", x, W, wv, wv2, ob, ob2, o32, T, W, 1e-6, 0, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_rmsnorm", x, W, wv, ob, o32, None, T, W, 1, 1e-6, 1, 1, None, 0, 0), 10)
        pair("two_norms_one_launch_vs_one_norm_2048_rows", t_new, t_old, (T * W * (4 + 2 + 2 + 4), T * W * (4 + 2 + 4)))
        y1, y2 = torch.randn(T, W, **f32), torch.randn(T, W, **f32)
        t_new = timed(lambda: _call("mrs_hyb_norm_pair_add", x, W, y1, wv, y2, wv2, T, W, 1e-6, 0.5, 1), 10)
        pair("normed_average_into_stream_vs_one_norm_2048_rows", t_new, t_old, (T * W * 16, T * W * (4 + 2 + 4)))
        E, top = z["experts"], z["top"]
        ids, wts, gt = torch.empty(T * top, dtype=torch.int32, device=dev), torch.empty(T * top, **f32), torch.empty(T, **f32)
        wr, br = torch.randn(E + 1, W, **f32), torch.randn(E, **f32)
        t_new = timed(lambda: _call("mrs_hyb_route_topk_softmax", x, wr, br, T, W, E, top, 1.0, ids, wts), 10)
        t_old = timed(lambda: _call("mrs_hyb_route_sigmoid_topk", x, wr, T, W, E, top, 0, ids, wts, gt), 10)
        pair("router_2048_rows", t_new, t_old, (T * W * 4 + E * W * 4, T * W * 4 + E * W * 4))
        ff = z["eff"]
        R_ = T * top
        up, gu = torch.randn(R_, ff, **f32), torch.randn(R_, 2 * ff, **f32)
        act = torch.empty(R_, ff, dtype=torch.bfloat16, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_relu_sq", up, act, R_, ff, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_glu_silu", gu, act, R_, ff, 1), 10)
        pair("expert_activation_prompt", t_new, t_old, (R_ * ff * 6, R_ * ff * 10))
        sp = cdel.s
        yv, gv, nw_ = torch.randn(T, cdel.nv, **f32), torch.randn(T, cdel.nv, **f32), torch.randn(cdel.nv, **f32)
        ov = torch.empty(T, cdel.nv, dtype=torch.bfloat16, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_head_norm_gate", yv, sp.vdim, None, nw_, 0, gv, cdel.nv, 1, ov, T, sp.heads, sp.vdim, 1e-6, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_rmsnorm", yv, cdel.nv, nw_, ov, None, None, T, cdel.nv, sp.heads, 1e-6, 0, 1, gv, cdel.nv, 0), 10)
        pair("head_norm_gate_vs_gated_group_norm_2048_rows", t_new, t_old, (T * cdel.nv * 10, T * cdel.nv * 10))
        # operands of the recurrence: convolution + unit vectors / write strengths / decays against convolution + step sizes
        uc = torch.randn(T, cdel.w_in.shape[0], **f32)
        cc = torch.empty(T, cdel.channels, **f32)
        av = torch.randn(T, sp.heads * cdel.per, **f32)
        beta, dec = torch.empty(T, sp.heads, **f32), torch.empty(T, sp.heads * cdel.per, **f32)

        def prep():
            _call("mrs_hyb_conv", uc, uc.stride(0), None, cdel.conv_w, None, cdel.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, cc, T, 1, cdel.channels, sp.conv, 1)
            _call("mrs_hyb_delta_prep", cc, cdel.channels, uc, uc.stride(0), cdel.b_col, av, av.stride(0), cdel.A_log, cdel.dt_bias, beta, dec, T, sp.heads, sp.kv_heads, sp.dim, cdel.per)
        ms = ossm_d.s
        uo = torch.randn(T, ossm_d.w_in.shape[0], **f32)
        xbc = torch.empty(T, ms.conv_channels, **f32)
        t_new = timed(prep, 10)
        t_old = timed(lambda: _call("mrs_hyb_conv_silu", uo[:, ms.inner:], uo.stride(0), ossm_d.conv_w, ossm_d.conv_b, ossm_d.conv_state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot,
                                    xbc, T, 1, ms.conv_channels, ms.conv), 10)
        pair("conv_and_delta_operands_vs_conv_2048_rows", t_new, t_old, (T * 4 * (2 * cdel.channels + 2 * 2 * cdel.nqk + 2 * sp.heads * cdel.per), T * 8 * ms.conv_channels), launches=3)
        nqkv = H * D + G * D + G * Dv
        uq = torch.randn(T, nqkv + H, **f32)
        ql = torch.empty(T, H * D, dtype=torch.bfloat16, device=dev)
        t_new = timed(lambda: _call("mrs_hyb_qk_headnorm_rope_cache", uq, nqkv + H, att.q_norm, att.k_norm, att.freq, b.tok_pos, b.slot_mapping, ql, att.k_cache, att.v_cache, T, H, G,
                                    D, Dv, D // 2, bs, 1e-6, 1), 10)
        t_old = timed(lambda: _call("mrs_hyb_qk_norm_rope_cache", uq, nqkv + H, oattn.q_norm, oattn.k_norm, oattn.freq, b.tok_pos, b.slot_mapping, ql, oattn.k_cache, oattn.v_cache, T, H,
                                    G, D, Dv, D // 2, bs, 1e-6, 1), 10)
        pair("head_norm_rotary_page_write_vs_whole_norm_rotary_page_write", t_new, t_old, (T * nqkv * 6, T * nqkv * 6))
    d1 = out["models"]["gifopel"]["decode"]["batch1"]
    print(json.dumps({"metric": "gifopel_decode_tokens_per_sec", "value": d1["tokens_per_sec"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": d1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"model": f"gifopel-{a.gifopel}", "global_batch": 1, "seq_len": 512, "parallelism": "tp1"}, "gifopel": out}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--batch", type=int, default=1, help="sequences decoded concurrently (1..8; BASELINE configs use 1): value = batch * steps / time")
    ap.add_argument("--shard-shapes", type=int, default=0, help="single GPU, no collectives: run ONE rank's shard shapes of a TP = N model (shape smoke test for --gpus N)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dropin", action="store_true", help="skip the drop-in launch sequence leg (dropin_tokens_per_sec)")
    ap.add_argument("--no-extra", action="store_true", help="skip the extra_configs legs (configs[2] ISQ Q8_0 and the configs[4] model on one GPU)")
    ap.add_argument("--parity-prompt", type=int, default=64, help="prompt length of the CPU-path parity leg (prefilled in one pass on both sides)")
    ap.add_argument("--small", action="store_true", help="tiny config (smoke / CI), not the benchmark")
    ap.add_argument("--tp", action="store_true", help="(default for N > 1) ONE model sharded tensor-parallel over the N GPUs")
    ap.add_argument("--replicas", action="store_true", help="N > 1: N independent replicas (weak scaling) instead of tensor parallelism")
    ap.add_argument("--model", choices=["auto", "8b", "70b", "mixtral"], default="auto",
                    help="auto: 70b (configs[3]) when N == 8, else 8b (configs[1]); mixtral: Mixtral-8x7B-shaped sparse MoE (configs[4]; TP = 2 with --gpus 2)")
    ap.add_argument("--weights", choices=["gaussian", "blocks"], default="gaussian",
                    help="gaussian (default): N(0, 0.02^2) through the device ISQ quantizers (SURVEY 8d); blocks: random valid block bytes (fast variant for pure kernel timing)")
    ap.add_argument("--parity-positions", type=int, default=16, help="greedy positions of the CPU-path parity leg")
    ap.add_argument("--quant", choices=["q4_k_m", "q8_0_isq"], default="q4_k_m",
                    help="q8_0_isq = BASELINE configs[2]: every linear quantized in situ from bf16 weights to Q8_0 on the GPU (mistralrs_amd.isq, role of generate_isq!)")
    ap.add_argument("--hybrid", choices=sorted(HYBRID_SIZES), default=None,
                    help="instead of the default workload: a layer-list decoder (state-space + windowed-attention mixers, routed experts; bf16) of the given size beside the Llama runner at equal size")
    ap.add_argument("--hybrid-no-llama", action="store_true", help="--hybrid: skip the equal-size Llama leg (profiling runs)")
    ap.add_argument("--hybrid-quick", action="store_true", help="--hybrid: the equal-size Llama leg at the short prompt only")
    ap.add_argument("--sobunex", choices=sorted(SOBUNEX_SIZES), default=None,
                    help="instead of the default workload: a Sobunex layer list (sigmoid attention with mixed head scores, dense / routed feed-forwards; bf16) of the given size beside "
                         "a windowed-attention + routed-experts list of the package at equal size, and the like kernels of the two one by one")
    ap.add_argument("--setopel", choices=sorted(SETOPEL_SIZES), default=None,
                    help="instead of the default workload: a Setopel layer list (residual streams; latent / sink attention, retention; SiLU-GLU feed-forwards; bf16) of the given size "
                         "beside an attention + state-space list of the package at equal size, and the like kernels of the two one by one")
    ap.add_argument("--gifopel", choices=sorted(GIFOPEL_SIZES), default=None,
                    help="instead of the default workload: a Gifopel layer list (matrix memory, chunked sink attention beside a delta rule, delta rule with channel decays; dense / routed "
                         "squared-ReLU feed-forwards; bf16) of the given size beside a state-space + windowed-attention + routed-experts list of the package at equal size, and the like "
                         "kernels of the two one by one")
    a = ap.parse_args()
    if a.gifopel:
        import torch
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        if a.steps == 256:
            a.steps = 128
        return gifopel_leg(a, dev)
    if a.setopel:
        import torch
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        if a.steps == 256:
            a.steps = 128
        return setopel_leg(a, dev)
    if a.sobunex:
        import torch
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        if a.steps == 256:
            a.steps = 128
        return sobunex_leg(a, dev)
    if a.hybrid:
        import torch
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        if a.steps == 256:
            a.steps = 128
        return hybrid_leg(a, dev)

    if a.gpus > 1 and "WORLD_SIZE" not in os.environ:
        # driver contract: `python bench.py --gpus N` must use N GPUs -- re-launch ourselves as one process per GPU (mistralrs-core/src/distributed.rs:569-795
        # spawns its ranks the same way)
        import socket
        import subprocess
        with socket.socket() as so:
            so.bind(("127.0.0.1", 0))
            port = so.getsockname()[1]
        cmd = [sys.executable, "-m", "torch.distributed.run", "--nnodes=1", f"--nproc-per-node={a.gpus}", "--master-addr", "127.0.0.1",
               "--master-port", str(port), os.path.abspath(__file__)] + sys.argv[1:]
        env = dict(os.environ, HSA_ENABLE_IPC_MODE_LEGACY=os.environ.get("HSA_ENABLE_IPC_MODE_LEGACY", "0"))
        sys.exit(subprocess.call(cmd, env=env))

    import torch
    import torch.distributed as dist
    if os.environ.get("MRS_BENCH_DRY_RUN"):
        # launcher check without GPUs (tests/test_distributed.py): every rank joins a gloo group, rank 0 prints the line's identity fields
        world = int(os.environ.get("WORLD_SIZE", "1"))
        if world > 1:
            dist.init_process_group("gloo")
            dist.barrier()
        tp = world > 1 and not a.replicas
        big = a.model == "70b" or (a.model == "auto" and world == 8 and not a.replicas)
        if int(os.environ.get("RANK", "0")) == 0:
            print(json.dumps({"metric": "decode_tokens_per_sec", "dry_run": True, "n_gpus": world, "steps": a.steps, "warmup": a.warmup,
                              "scaling": "strong" if tp else "weak",
                              "config": {"workload": ("Llama-3-70B" if big else "Llama-3-8B") + " GGUF Q4_K_M", "parallelism": "tp1" if world == 1 else (f"tp{world}" if tp else f"replicas x{world}")}}), flush=True)
        if world > 1:
            dist.destroy_process_group()
        return
    rank = int(os.environ.get("RANK", "0"))
    local_rank = int(os.environ.get("LOCAL_RANK", "0"))
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if world != a.gpus and rank == 0:
        print(f"bench.py: --gpus {a.gpus} but WORLD_SIZE={world}: measuring {world} rank(s)", file=sys.stderr)
    if world > 1:
        torch.cuda.set_device(local_rank)
        dist.init_process_group("nccl", device_id=torch.device("cuda", local_rank))
    dev = torch.device("cuda", local_rank if world > 1 else 0)
    torch.cuda.set_device(dev)

    import mistralrs_amd  # noqa: F401
    from mistralrs_amd.llama import LlamaConfig
    big = a.model == "70b" or (a.model == "auto" and world == 8 and not a.replicas)
    if big and a.prompt_len == 512:
        a.prompt_len = 2048  # configs[3]: 2048 prefill / 256 decode
    BATCH_LEG = (8, 64)  # warm-up / timed steps of the batched_decode side leg: the model is sized for it whatever --steps says
    leg_steps = max(a.warmup + a.steps, sum(BATCH_LEG))
    ctx_needed = a.prompt_len + leg_steps + 2
    max_ctx = (ctx_needed + 63) // 64 * 64
    if a.small:
        cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_layers=2, num_heads=8, num_kv_heads=2, vocab_size=2048,
                          head_dim=64, max_batch=8, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        name = "tiny-llama (smoke)"
    elif a.model == "mixtral":
        cfg = LlamaConfig.mixtral_8x7b(max_batch=8, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        name = "Mixtral-8x7B-shaped (8 experts, top-2)"
    elif big:
        cfg = LlamaConfig.llama3_70b(max_batch=8, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        name = "Llama-3-70B"
    else:
        cfg = LlamaConfig.llama3_8b(max_batch=8, max_context_len=max_ctx, max_position_embeddings=max(8192, max_ctx))
        name = "Llama-3-8B"
    if a.shard_shapes > 1 and world == 1:
        from mistralrs_amd import distributed as D
        cfg.num_heads, cfg.num_kv_heads, cfg.intermediate_size = D.local_dims(cfg.num_heads, cfg.num_kv_heads, cfg.intermediate_size, a.shard_shapes)
        name += f" (shapes of one rank of TP={a.shard_shapes}, no collectives)"
    tp = world > 1 and not a.replicas
    if tp:  # column / row parallel shards (mistralrs-quant/src/distributed/layers.rs): local heads, kv heads, ffn
        from mistralrs_amd import distributed as D
        cfg.head_dim = cfg.head_dim  # keep the global head_dim
        cfg.num_heads, cfg.num_kv_heads, cfg.intermediate_size = D.local_dims(cfg.num_heads, cfg.num_kv_heads, cfg.intermediate_size, world)
        cfg.tp_world_size, cfg.tp_rank = world, rank
    model = build_model(cfg, dev, seed=0 if tp else rank, max_new_tokens=leg_steps + 8, tp=(rank, world) if tp else None, quant=a.quant, weights=a.weights)
    comm, p2p = None, None
    if tp:
        from mistralrs_amd import distributed as D
        comm = D.RcclComm(rank, world, dev)
        assert comm.nranks() == world, f"RCCL communicator has {comm.nranks()} ranks, expected {world}"
        model.set_comm(comm)
        # decode-sized all-reduces: one-shot peer-mailbox route (csrc/ext_p2p.hip) when it is available AND agrees with RCCL on a probe vector on
        # every rank; otherwise RCCL carries everything
        p2p, p2p_note = None, "rccl only"
        if not os.environ.get("MRS_NO_P2P"):
            try:
                p2p = D.P2PAllReduce(rank, world, dev)
                probe = (torch.arange(4096, device=dev, dtype=torch.float32) % 97) * (rank + 1)
                a1, a2 = probe.clone(), probe.clone()
                p2p.all_reduce_(a1)
                comm.all_reduce_(a2)
                torch.cuda.synchronize()
                good = torch.tensor([int(torch.equal(a1, a2) and p2p.error() == 0)], device=dev)
            except Exception as e:  # IPC not available on this box
                good, p2p_note = torch.tensor([0], device=dev), f"rccl only (p2p unavailable: {type(e).__name__})"
            dist.all_reduce(good, op=dist.ReduceOp.MIN)
            if int(good.item()) == 1:
                model.set_p2p(p2p)
                p2p_note = "one-shot peer-mailbox all-reduce over xGMI (ext_p2p.hip) for [1, hidden]; RCCL for the prefill messages"
            else:
                p2p = None
    torch.cuda.synchronize()

    def sync():
        if world > 1:
            dist.barrier()
        torch.cuda.synchronize()

    r = timed_run(model, cfg, a.prompt_len, a.steps, a.warmup, a.batch, sync, world, dev)
    if tp and p2p is not None:
        # the peer-mailbox route reports a granule that never arrived through its error word (bounded spin, NaN sums): if ANY rank saw one, every rank drops
        # the route and the whole timed pass is repeated on RCCL -- a number measured over NaN sums is not a measurement
        if model.p2p_sync_error():  # MAX over the ranks, every rank detaches in the same step (mrs_hip_ext.h: mrs_llama_check_p2p)
            p2p, p2p_note = None, "rccl only (the p2p route raised its error word during the timed pass: dropped, pass repeated on RCCL)"
            r = timed_run(model, cfg, a.prompt_len, a.steps, a.warmup, a.batch, sync, world, dev)
    prompt, ttft, prefill_flops, B, t_all, dev_s, toks = r["prompt"], r["ttft"], r["prefill_flops"], r["B"], r["t_all"], r["dev_s"], r["toks"]
    prefill_exact = bool(model.prefill_is_exact)
    ttft_bf16, ttft_bf16_fused = None, None
    if prefill_exact and world == 1:  # the same prompt through the bf16-operand MFMA GEMMs + flash attention (selectable: Llama.set_prefill_mode(0) / MRS_PREFILL_EXACT=0)
        def timed_prefill(mode):
            model.set_prefill_mode(mode)
            model.prefill(prompt, 0, seq=min(1, cfg.max_batch - 1))
            sync()
            t0 = time.perf_counter()
            int(model.prefill(prompt, 0, seq=min(1, cfg.max_batch - 1)).argmax())
            return time.perf_counter() - t0
        ttft_bf16 = timed_prefill(0)  # library bf16 GEMMs on the bf16 shadow copy of the weights when the model has one (csrc/ext_gemm_lt.hip), else the fused block dequant
        if model.bf16_shadow:
            ttft_bf16_fused = timed_prefill(2)  # A / B: the fused block-dequant -> bf16 MFMA kernels of rounds 2-5 on the same prompt
        model.set_prefill_mode(-1)

    # ---------------- roofline of the dominant kernel: the decode engine's gate/up phase (RMSNorm + Q8_K quantize + 2 x [ffn, d] GEMV + SiLU*up),
    # timed with HIP events on the launch stream over every layer's weights (>= 1 GB: nothing Infinity-Cache resident)
    import ctypes as C
    from mistralrs_amd import _lib
    ext = _lib.load("ext")

    class Mat(C.Structure):
        _fields_ = [("planes", C.c_void_p), ("type", C.c_int), ("n", C.c_longlong), ("k", C.c_longlong)]
    MP = C.POINTER(Mat)
    ext.mrs_dec_gate_up.argtypes = [MP, MP, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_float, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    h = torch.randn(1, cfg.hidden_size, device=dev)
    act = torch.empty(1, cfg.intermediate_size, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    assert model.decode_path == "engine", model.decode_path
    layers = []
    moe = cfg.num_experts > 0
    sfx = "_exps" if moe else ""
    for i in range(cfg.num_layers):
        g, u = model._keep[f"blk.{i}.ffn_gate{sfx}.weight"], model._keep[f"blk.{i}.ffn_up{sfx}.weight"]
        layers.append((Mat(model._keep[f"blk.{i}.ffn_gate{sfx}.weight#dec"].data_ptr(), g.dtype.id, g.shape[0], g.shape[1]),
                       Mat(model._keep[f"blk.{i}.ffn_up{sfx}.weight#dec"].data_ptr(), u.dtype.id, u.shape[0], u.shape[1]),
                       model._keep[f"blk.{i}.ffn_norm.weight"], (g.nbytes() + u.nbytes()) * (cfg.num_experts_per_tok / cfg.num_experts if moe else 1)))
    if moe:  # the top-k experts' gate / up rows in ONE launch (mrs_dec_gate_up_topk); expert ids on the device
        ext.mrs_dec_gate_up_topk.argtypes = [MP, MP, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        sel = torch.tensor([1, 5][: cfg.num_experts_per_tok], dtype=torch.int32, device=dev)
        act = torch.empty(cfg.num_experts_per_tok, cfg.intermediate_size, device=dev)

    def gate_up_pass():
        for mg, mu, nw, _ in layers:
            if moe:
                rc = ext.mrs_dec_gate_up_topk(C.byref(mg), C.byref(mu), cfg.intermediate_size, sel.data_ptr(), cfg.num_experts_per_tok, h.data_ptr(), nw.data_ptr(), cfg.rms_eps, 0,
                                              act.data_ptr(), cfg.intermediate_size, st)
            else:
                rc = ext.mrs_dec_gate_up(C.byref(mg), C.byref(mu), cfg.intermediate_size, None, h.data_ptr(), cfg.hidden_size, nw.data_ptr(), cfg.rms_eps, 0,
                                         act.data_ptr(), cfg.intermediate_size, 1, st)
            assert rc == 0
    gate_up_pass()
    torch.cuda.synchronize()
    reps = 8
    k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    k0.record()
    for _ in range(reps):
        gate_up_pass()
    k1.record()
    torch.cuda.synchronize()
    kern_s = k0.elapsed_time(k1) / 1e3 / (reps * len(layers))
    kern_bytes = int(layers[0][3])  # algorithmic bytes per launch: the two GGUF weight tensors (the decode layout holds the same bits + 2.8 % for 8-bit scales)
    achieved = kern_bytes / kern_s

    # ---------------- tensor parallel: cost of the decode all-reduces (2 per layer, [1, hidden] f32) measured on the same communicator
    ar = None
    if tp:
        buf = torch.zeros(cfg.hidden_size, device=dev)
        for _ in range(10):
            comm.all_reduce_(buf)
        sync()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(200):
            comm.all_reduce_(buf)
        e1.record()
        sync()
        us = e0.elapsed_time(e1) * 1e3 / 200
        ar = {"rccl_us_per_call": round(us, 2), "calls_per_step": 2 * cfg.num_layers, "bytes": cfg.hidden_size * 4, "decode_route": p2p_note}
        if p2p is not None:
            for _ in range(10):
                p2p.all_reduce_(buf)
            sync()
            e0.record()
            for _ in range(200):
                p2p.all_reduce_(buf)
            e1.record()
            sync()
            ar["p2p_us_per_call"] = round(e0.elapsed_time(e1) * 1e3 / 200, 2)
        used = ar.get("p2p_us_per_call", ar["rccl_us_per_call"])
        ar["frac_of_step"] = round(used * 2 * cfg.num_layers / (1e6 * t_all / a.steps), 4)  # back-to-back launches; in the step they sit inside the captured graph

    avg_ctx = a.prompt_len + a.warmup + a.steps / 2
    step_bytes = model.decode_bytes(B, int(avg_ctx))
    tok_s = (1 if tp else world) * B * a.steps / t_all  # TP: the N GPUs decode ONE sequence (B sequences with --batch)
    out = {
        "metric": "decode_tokens_per_sec", "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": world, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(1e3 * t_all / a.steps, 4), "higher_is_better": True, "scaling": "strong" if tp else "weak",
        "vs_baseline": None, "dtype": ("q4_k/q6_k weights x q8_k activations" if a.quant == "q4_k_m" else "q8_0 weights x q8_0 activations") + " (int8 dot, f32 accumulate: the reference CPU path's arithmetic)", "data": "synthetic",
        "config": {"workload": f"{name} " + ("GGUF Q4_K_M" if a.quant == "q4_k_m" else "ISQ Q8_0 (in situ from bf16, on the GPU)") + f", TP={world if tp else 1}, {a.prompt_len} prefill / {a.steps} decode, batch {B}, paged KV bf16 (block 32)",
                   "parallelism": "tp1" if world == 1 else (f"tp{world}" if tp else f"replicas x{world}")},
        "prefill_tokens_per_sec": round(a.prompt_len / ttft, 1), "ttft_ms": round(1e3 * ttft, 2),
        "prefill_arithmetic": ("decode engine's: Q8_K activation rows x exact-integer f16 MFMA block dots, one f32 term per superblock (mrs_gemm_qi), decode attention per query "
                               "-- logits and KV pages identical to token-by-token decode" if prefill_exact else "bf16-operand MFMA (fused block dequant) + MFMA flash attention"),
        "prefill_roofline": {"bound": "mfma", "achieved": round(prefill_flops / ttft / 1e12, 1), "peak": MFMA_PEAK / 1e12, "unit": "TFLOP/s",
                             "frac": round(prefill_flops / ttft / MFMA_PEAK, 4), "flops": prefill_flops,
                             "note": ("exact-integer f16 MFMA GEMMs on Q8_K activation images (mrs_gemm_qi) + per-query decode attention over the paged cache"
                                      if prefill_exact else "fused block-dequant -> bf16 MFMA GEMMs (mrs_gemm_q_bf16_multi) + MFMA flash attention over the paged cache")
                                     + "; whole prompt incl. the host read-back of the first token"},
        "device_ms_per_step": round(1e3 * dev_s / a.steps, 4),
        "step_bytes": int(step_bytes), "step_roofline_frac": round(step_bytes * (a.steps / t_all) / HBM_PEAK, 4),
        # `frac` is what THIS process measured: HIP events on the launch stream around back-to-back launches of the kernel over every layer's weights (2.1 GB: nothing
        # cache-resident).  The in-graph average of the committed rocprofv3 trace (launch boundary included) is the side object `in_graph`, quoted only when the profile
        # was taken from this very build (source digest).
        "roofline": {"bound": "hbm", "kernel": "dec_gemv_kernel<1, EPI_GLU> (decode engine gate/up phase: RMSNorm + Q8_K quantize + gate/up GEMV + SiLU*up)",
                     "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4),
                     "bytes_per_launch": int(kern_bytes), "us_per_launch": round(kern_s * 1e6, 2),
                     "frac_source": "live: HIP events on the launch stream over back-to-back launches of every layer's weights, this process", "source_digest": source_digest(),
                     **committed_profile(name, a.quant)},
        "greedy_tokens_head": [int(t) for t in toks[a.warmup: a.warmup + 8]],
    }
    rl = out["roofline"]
    if rl.get("in_graph"):
        rl["in_graph"]["achieved"] = round(kern_bytes / (rl["in_graph"]["us_per_launch"] * 1e-6) / 1e9, 1)
        rl["in_graph"]["frac"] = round(kern_bytes / (rl["in_graph"]["us_per_launch"] * 1e-6) / HBM_PEAK, 4)
    if ttft_bf16 is not None:
        out["prefill_bf16"] = {"tokens_per_sec": round(a.prompt_len / ttft_bf16, 1), "ttft_ms": round(1e3 * ttft_bf16, 2), "frac": round(prefill_flops / ttft_bf16 / MFMA_PEAK, 4),
                               "gemm": ("hipBLASLt bf16 x bf16 -> f32 on a bf16 shadow copy of the dense linears (dequantized once at load: 2 bytes per weight)" if model.bf16_shadow
                                        else "fused block dequant -> bf16 MFMA (mrs_gemm_q_bf16_multi)"),
                               **({"fused_dequant_kernels": {"tokens_per_sec": round(a.prompt_len / ttft_bf16_fused, 1), "ttft_ms": round(1e3 * ttft_bf16_fused, 2),
                                                             "frac": round(prefill_flops / ttft_bf16_fused / MFMA_PEAK, 4)}} if ttft_bf16_fused else {}),
                               "note": "same prompt through the selectable bf16-operand path (Llama.set_prefill_mode(0) / MRS_PREFILL_EXACT=0): faster, but its logits and KV pages are "
                                       "only close to (not identical with) the decode engine's -- the default keeps the reference CPU arithmetic"}
    if ar is not None:
        out["allreduce"] = ar
    if world == 1 and B == 1 and not a.no_dropin and not a.small and a.quant == "q4_k_m" and not moe:
        try:
            d_tok, d_frac = dropin_rate(model, cfg, prompt, min(a.steps, 64), dev)
            out["dropin_tokens_per_sec"] = round(d_tok, 2)
            out["dropin_step_roofline_frac"] = round(d_frac, 4)
            out["dropin_note"] = "the reference's own launch sequence through the drop-in C ABI (use_fused = 0: ~16 launches per layer, Q8_1 activations) -- what an unmodified Rust host gets; value / step_roofline_frac above are the MI355X-native engine (C++ runner)"
        except Exception as e:
            out["dropin_tokens_per_sec"] = None
            out["dropin_note"] = f"failed: {e}"
    if rank == 0 and world == 1 and not a.no_cpu_baseline:
        try:
            out["cpu_baseline"], par = parity_leg(model, cfg, a, prefill_exact)
            out.update(par)
        except Exception as e:  # the baseline is a reported extra, never fatal
            import traceback
            out["cpu_baseline"] = {"value": None, "unit": "tokens/s", "cores": 0, "kind": "port", "sample": f"failed: {e}: {traceback.format_exc()[-400:]}"}
    if rank == 0 and world == 1 and not a.no_extra and not a.small and B == 1 and a.quant == "q4_k_m" and not moe and cfg.max_batch >= 8 and not a.shard_shapes:
        # side field, never fatal: the same model decoding 4 and 8 sequences per step (the reference's MMVQ contract: batch 1-8 from one weight pass, mmvq_gguf.cu:724-792;
        # what the scheduler feeds).  `value` stays the batch-1 line BASELINE.json names.
        try:
            bw, bs_ = BATCH_LEG
            out["batched_decode"] = {"note": f"same weights, b sequences per step (same prompt in b sets of pages), {bs_} timed steps after {bw} warm-up steps; tokens/s = b * steps / time"}
            for bb in (2, 4, 8):
                rb = timed_run(model, cfg, a.prompt_len, bs_, bw, bb, sync, world, dev)
                out["batched_decode"][str(bb)] = {"tokens_per_sec": round(bb * bs_ / rb["t_all"], 2), "ms_per_step": round(1e3 * rb["t_all"] / bs_, 4),
                                                  "step_roofline_frac": round(model.decode_bytes(bb, int(a.prompt_len + bw + bs_ / 2)) * (bs_ / rb["t_all"]) / HBM_PEAK, 4)}
        except Exception as e:
            out["batched_decode"] = {"failed": f"{type(e).__name__}: {e}"}
    if rank == 0 and world == 1 and not a.no_extra and not a.small and B == 1 and a.quant == "q4_k_m" and a.model in ("auto", "8b") and not a.shard_shapes:
        out["extra_configs"] = {}
        del model
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        for kind in ("q8_0_isq", "mixtral", "70b"):
            try:
                out["extra_configs"][kind] = extra_config(kind, dev)
            except Exception as e:
                out["extra_configs"][kind] = {"failed": f"{type(e).__name__}: {e}"}
    if rank == 0:
        print(json.dumps(out), flush=True)
    if world > 1:
        dist.destroy_process_group()


if __name__ == "__main__":
    main()
