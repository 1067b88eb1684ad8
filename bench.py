"""Benchmark of the pair-stack block (triangle multiplication out + in, triangle attention
start + end, residual adds fused) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--n 768] [--no-cpu]

A step is one block forward on a z that already lives in HBM; every step reads the same input (the
result goes to a tensor of the block's own, so the data-dependent branches of the kernels see the
same data in every step).  The workload is benchmark configuration 3: N_token = 768, c_z = 128, c_hidden_mul = 128, 4 heads x 32, batch 1,
all-ones mask, bf16, synthetic N(0,1) input and seeded random weights.  Prints one JSON line.

Besides the whole-block time (`value`: wall clock over the K steps; `step_ms_median` / `step_ms_min`:
one event pair per step in a second loop of K steps; `inplace_ms_per_step`: the same loop run in place
with inplace_safe, where z drifts from step to step, for comparison) the line carries
  roofline      the triangle-multiplication contraction (the MFMA-bound kernel the target
                of >= 50 % of bf16 peak is set on): algorithmic 2*B*N^3*C_h flops over its
                average launch duration, measured here with events on the launch stream;
  kernels       the same figure for every kernel of the block (average over its launches in
                the block: both directions of each module), each against the roof that
                bounds it (MFMA for the contraction and the attention core, HBM for the
                LayerNorm/projection passes; algorithmic bytes per launch are listed in
                KERNEL_MODEL below);
                the entries "pair_transition" (the SwiGLU transition that follows the block in
                every PairBlock) and "pair_bias_proj" (the 16-head pair bias the single-representation
                attention of a PairFormerBlock takes from z), "attn_pair_bias" (that attention itself
                over s [N, 384], 16 heads of 24: its three small kernels as one call), "single_transition"
                (the SwiGLU transition of s, n = 4: two small kernels as one call) and "template_tail" (closing LayerNorm
                of the template stack, mean over 4 templates, ReLU and linear_t, c_t = 64 -> c_z
                = 128, at the same N) are timed right after the block's kernels and are not part
                of `value`;
  pairformer_block_ms  wall clock of one whole PairFormerBlock (of3pair.PairFormerBlock: the pair-stack
                block plus pair transition, pair bias, attention over s and single transition) at
                the same N, for orientation; not part of `value`;
  fp32_block_ms  wall clock of the same pair-stack block in fp32 (the reference's default inference
                precision; of3pair.PairStack on fp32 tensors), for orientation; not part of `value`;
  fp32_pairformer_block_ms  wall clock of the whole PairFormerBlock in fp32, for orientation;
  template_block_ms  {"bf16", "fp32"}: wall clock of one block of the template pair stack (of3pair.PairBlock,
                4 templates, N = 512, c_t = 64, 4 heads x 16, transition n = 2, padded tails: the benchmark's
                fourth configuration whatever --n says), for orientation;
  configs       the benchmark's configurations 2, 4 and 5 (N = 384 with a padded tail; the 2-block template
                pair stack over 4 templates at N = 512, c_t = 64, 4 x 16; 4 stacked blocks in place at N = 2048):
                wall clock through the modules ("ms", "ms_per_block") and the block's six kernels against their
                roofs, measured like `kernels`; not part of `value` (--configs '' leaves them out);
  cpu_baseline  the CPU oracle (fp32 PyTorch restatement of the reference's stock path) on the host
                cores for the same workload: one warm-up run, then the median of three.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "openfold-3_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

CAL_BYTES = 256 << 20      # size of the calibration copy

# HBM bytes per launch of the contraction at the headline workload (N=768, B=1), from two
# counter passes of this command (rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE), each
# scaled by what the same counter reads for the calibration copy; the summaries are kept in
# profiles/.  Keyed by (N, tile variant the library picks for that shape): a figure measured
# on one kernel variant is not reported for another; None for any other workload.
MEASURED_TRAFFIC = {(768, 1): 539701909, (768, 4): 500769092}

TRANSITION_N = 4           # hidden width factor of the pair transition (AF3 configuration)
PAIR_BIAS_HEADS = 16       # heads of the pairformer's single-representation attention
TEMPLATES, C_T = 4, 64     # templates and template channels of the AF3 configuration
C_S, C_HEAD_S = 384, 24    # single representation and head width of its attention

METRIC = "ms per Pairformer pair-stack block at N=768 bf16; % of MFMA peak & HBM GB/s"


def kernel_model(B, N, C, CH, H, D, transition_n=None):
    """Algorithmic work per launch.  U = one bf16 pass over z."""
    transition_n = TRANSITION_N if transition_n is None else transition_n
    U = B * N * N * C * 2
    hd = H * D
    return {
        # reads z, writes a and b
        "trimul_proj": {"bound": "hbm", "bytes": U + 2 * B * N * N * CH * 2 + B * N * N * 4},
        # 2*B*N^3*C_h multiply-adds counted as 2 flops
        "trimul_contract": {"bound": "mfma", "flops": 2 * B * N ** 3 * CH},
        # reads x and z, writes out
        "trimul_out": {"bound": "hbm", "bytes": B * N * N * CH * 2 + 2 * U},
        # reads x, writes q, k, v (+ fp32 triangle bias and mask bias)
        "triattn_proj": {"bound": "hbm", "bytes": U + 3 * B * N * N * hd * 2 + B * H * N * N * 4 + B * N * N * 4},
        # QK^T and PV
        "triattn_flash": {"bound": "mfma", "flops": 4 * B * N ** 3 * H * D},
        # reads o and x, writes out
        "triattn_out": {"bound": "hbm", "bytes": B * N * N * hd * 2 + 2 * U},
        # the transition after the block (n = 4): three C x 4C products per position
        "pair_transition": {"bound": "mfma", "flops": 6 * B * N * N * C * (transition_n * C)},
        # reads z, writes the [PAIR_BIAS_HEADS, N, N] bias
        "pair_bias_proj": {"bound": "hbm", "bytes": U + B * PAIR_BIAS_HEADS * N * N * 2},
        # LayerNorm + q, k, v, g projections, QK^T and PV over 16 heads of 24, output projection
        "attn_pair_bias": {"bound": "mfma", "flops": 10 * B * N * C_S * C_S + 4 * B * N * N * C_S},
        # three C_s x 4 C_s products per token
        "single_transition": {"bound": "mfma", "flops": 6 * B * N * C_S * (TRANSITION_N * C_S)},
        # reads the TEMPLATES planes of c_t channels, writes one c_z plane
        "template_tail": {"bound": "hbm", "bytes": B * N * N * 2 * (TEMPLATES * C_T + C)},
    }


def block_stage_launches(lib, _lib, torch, dp, zz, mask, dims, contract_variant=0):
    """The pair-stack block issued kernel by kernel through the stage entry points of the C ABI, in the
    order the block runs them (trimul out, trimul in, tri-attn start, tri-attn end), in place on zz.
    dp: device parameters under the PairStack names; returns [(kernel name, launch function)] and the
    intermediates and stride arrays that have to stay alive."""
    B, N, C, CH, H, D = dims
    dev, bf = zz.device, torch.bfloat16
    s = torch.cuda.current_stream().cuda_stream
    Np = lib.of3_padded_n(N)
    sb, si, sj = zz.stride()[:3]
    z_fwd, z_tr = _lib.strides3((sb, si, sj)), _lib.strides3((sb, sj, si))
    mb_, mi, mj = mask.stride()
    m_fwd, m_tr = _lib.strides3((mb_, mi, mj)), _lib.strides3((mb_, mj, mi))
    a = torch.zeros(B, CH, Np, Np, dtype=bf, device=dev)
    b = torch.zeros_like(a)
    x = torch.zeros_like(a)
    q = torch.zeros(B, N, H, Np, D, dtype=bf, device=dev)
    k = torch.zeros_like(q)
    vt = torch.zeros(B, N, H, D, Np, dtype=bf, device=dev)
    tb = torch.zeros(B, H, N, Np, device=dev)
    mb = torch.zeros(B, N, Np, device=dev)
    o = torch.zeros(B, N, N, H * D, dtype=bf, device=dev)
    P = lambda t: t.data_ptr()  # noqa: E731

    def ck(st):
        _lib.check(st, "bench stage")

    def trimul(prefix, outgoing):
        w = lambda name: P(dp[prefix + name])  # noqa: E731
        return [
            ("trimul_proj", lambda: ck(lib.of3_trimul_proj(
                P(zz), z_fwd, P(mask), m_fwd, w("layer_norm_in.weight"), w("layer_norm_in.bias"),
                w("linear_a_p.weight"), w("linear_a_g.weight"), w("linear_b_p.weight"), w("linear_b_g.weight"),
                P(a), P(b), B, N, C, CH, outgoing, s))),
            ("trimul_contract", lambda: ck(lib.of3_trimul_contract(P(a), P(b), P(x), B, N, CH, contract_variant, s))),
            ("trimul_out", lambda: ck(lib.of3_trimul_out(
                P(x), P(zz), z_fwd, P(zz), w("layer_norm_in.weight"), w("layer_norm_in.bias"),
                w("layer_norm_out.weight"), w("layer_norm_out.bias"), w("linear_g.weight"), w("linear_z.weight"),
                B, N, C, CH, 1, s))),
        ]

    def triattn(prefix, zs, ms_):
        w = lambda name: P(dp[prefix + name])  # noqa: E731
        return [
            ("triattn_proj", lambda: ck(lib.of3_triattn_proj(
                P(zz), zs, P(mask), ms_, w("layer_norm.weight"), w("layer_norm.bias"), w("mha.linear_q.weight"),
                w("mha.linear_k.weight"), w("mha.linear_v.weight"), w("linear_z.weight"),
                P(q), P(k), P(vt), P(tb), P(mb), B, N, C, H, D, 1e9, s))),
            ("triattn_flash", lambda: ck(lib.of3_triattn_flash(P(q), P(k), P(vt), P(tb), P(mb), P(o), B, N, H, D, s))),
            ("triattn_out", lambda: ck(lib.of3_triattn_out(
                P(o), P(zz), zs, P(zz), w("layer_norm.weight"), w("layer_norm.bias"), w("mha.linear_g.weight"),
                w("mha.linear_o.weight"), B, N, C, H, D, 1, s))),
        ]

    stage_list = (trimul("tri_mul_out.", 1) + trimul("tri_mul_in.", 0)
                  + triattn("tri_att_start.", z_fwd, m_fwd) + triattn("tri_att_end.", z_tr, m_tr))
    return stage_list, (a, b, x, q, k, vt, tb, mb, o, z_fwd, z_tr, m_fwd, m_tr)


def time_launches(torch, launches, steps, warmup):
    """Every launch bracketed by its own pair of events on the launch stream: {name: [ms per launch]}."""
    for _ in range(max(warmup, 1)):
        for _, fn in launches:
            fn()
    torch.cuda.synchronize()
    marks = []
    for _ in range(steps):
        for name, fn in launches:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            marks.append((name, e0, e1))
    torch.cuda.synchronize()
    durations = {}
    for name, e0, e1 in marks:
        durations.setdefault(name, []).append(e0.elapsed_time(e1))
    return durations


def kernel_figures(durations, model):
    """Mean launch duration of every kernel against the roof that bounds it."""
    kernels = {}
    for name, vals in durations.items():
        ms = sum(vals) / len(vals)
        m = model[name]
        if m["bound"] == "mfma":
            ach = m["flops"] / (ms * 1e-3) / 1e12
            kernels[name] = {"bound": "mfma", "ms": round(ms, 4), "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS,
                             "unit": "TFLOP/s", "frac": round(ach / PEAK_BF16_TFLOPS, 4)}
        else:
            ach = m["bytes"] / (ms * 1e-3) / 1e9
            kernels[name] = {"bound": "hbm", "ms": round(ms, 4), "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4)}
    return kernels


def other_configs(of3pair, lib, _lib, orc, torch, dev, which):
    """The benchmark's configurations 2, 4 and 5 (configuration 3 is `value`; configuration 1 is the CPU
    plumbing case): wall clock through the module interface and the block's six kernels one by one, each
    against its roof.  Not part of `value`.

      2  one pair-stack block, B = 1, N = 384, c_z = 128, the last 10 % of the tokens masked
      4  the template pair stack: 2 TemplatePairBlocks (pair stack + transition n = 2) over 4 templates,
         N = 512, c_t = 64, 4 heads x 16, per-template padding of 0-20 %
      5  4 stacked pair-stack blocks in place at N = 2048, c_z = 128, the last 256 tokens masked
    """
    bf = torch.bfloat16
    out = {}

    def wall(fn, reps, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps

    def stage_figures(params, zz, mask, dims, reps, warm):
        dp = {k_: v.to(dev).to(bf).contiguous() for k_, v in params.items()}
        stage_list, keep = block_stage_launches(lib, _lib, torch, dp, zz, mask, dims)
        fig = kernel_figures(time_launches(torch, stage_list, reps, warm), kernel_model(*dims))
        del stage_list, keep
        return fig

    if 2 in which:
        B, N, C, CH, H, D = dims = (1, 384, 128, 128, 4, 32)
        params = {k_: orc.round_bf16(v) for k_, v in orc.make_block_params(0, C, CH, D, H).items()}
        blk = of3pair.PairStack(C, CH, D, H)
        blk.load_state_dict(params)
        blk = blk.to(dev).to(bf).eval()
        z = orc.round_bf16(orc.make_pair_input(2, (B,), N, C)).to(dev).to(bf)
        mask = orc.tail_padding_mask((B,), N, N // 10).to(dev)
        ms = wall(lambda: blk(z, mask), 30, 10)
        out["2"] = {"workload": "pair-stack block, B=1, N_token=384, c_z=128, last 10% of tokens masked",
                    "blocks": 1, "ms": round(ms, 4), "ms_per_block": round(ms, 4),
                    "kernels": stage_figures(params, z.clone(), mask, dims, 20, 5)}
        del blk, z, mask
    if 4 in which:
        B, N, C, CH, H, D = dims = (4, 512, 64, 64, 4, 16)
        gen = torch.Generator().manual_seed(3)
        sd, first = {}, None
        for i in range(2):
            bp = dict(orc.make_block_params(30 + i, C, CH, D, H))
            bp.update({"pair_transition." + k_: v for k_, v in orc.make_transition_params(gen, C, 2).items()})
            bp = {k_: orc.round_bf16(v) for k_, v in bp.items()}
            first = first or bp
            sd.update({"blocks.%d.%s" % (i, k_): v for k_, v in bp.items()})
        sd["layer_norm.weight"], sd["layer_norm.bias"] = torch.ones(C), torch.zeros(C)
        stack = of3pair.TemplatePairStack(c_t=C, c_hidden_tri_att=D, c_hidden_tri_mul=CH, no_blocks=2, no_heads=H,
                                          pair_transition_n=2, dropout_rate=0.25, tri_mul_first=True)
        stack.load_state_dict(sd, strict=True)
        stack = stack.to(dev).to(bf).eval()
        t = orc.round_bf16(orc.make_pair_input(3, (B,), N, C)).to(dev).to(bf)
        mask = orc.tail_padding_mask((B,), N, torch.tensor([0, 20, 51, 102])).to(dev)
        ms = wall(lambda: stack.run_blocks(t, mask), 10, 3)
        out["4"] = {"workload": "template pair stack: 2 blocks (pair stack + transition n=2), 4 templates, N_token=512, "
                                "c_t=64, c_hidden_mul=64, 4 heads x 16, per-template padding 0-20%",
                    "blocks": 2, "ms": round(ms, 4), "ms_per_block": round(ms / 2, 4),
                    "kernels": stage_figures(first, t.clone(), mask, dims, 10, 3)}
        del stack, t, mask
    if 5 in which:
        B, N, C, CH, H, D = dims = (1, 2048, 128, 128, 4, 32)
        blocks, params = [], None
        for i in range(4):
            params = {k_: orc.round_bf16(v) for k_, v in orc.make_block_params(50 + i, C, CH, D, H).items()}
            blk = of3pair.PairStack(C, CH, D, H)
            blk.load_state_dict(params)
            blocks.append(blk.to(dev).to(bf).eval())
        z0 = torch.randn(B, N, N, C, generator=torch.Generator().manual_seed(5)).to(bf).to(dev)
        mask = orc.tail_padding_mask((B,), N, 256).to(dev)
        zw = torch.empty_like(z0)

        def four_blocks():
            zw.copy_(z0)  # the stack runs in place on a fresh copy (a 1 GB device copy, counted: ~0.4 ms of ~100)
            zz = zw
            for blk_ in blocks:
                zz = blk_(zz, mask, inplace_safe=True)

        ms = wall(four_blocks, 3, 1)
        del blocks
        from of3pair import functional as F3
        F3.release_workspaces()
        torch.cuda.empty_cache()
        fig = stage_figures(params, zw, mask, dims, 3, 1)
        out["5"] = {"workload": "4 stacked pair-stack blocks in place, B=1, N_token=2048, c_z=128, last 256 tokens "
                                "masked (~1 GB pair representation)",
                    "blocks": 4, "ms": round(ms, 3), "ms_per_block": round(ms / 4, 3), "kernels": fig}
        del z0, zw, mask
    torch.cuda.empty_cache()
    return out


def extra_legs(of3pair, orc, pf, s_pf, z32, sm, m32, fp32_reps, dev):
    """Legs beside the headline workload, wall clock, informative: the whole PairFormerBlock in fp32 and one
    block of the template pair stack at its own shape in both precisions."""
    import torch

    bf = torch.bfloat16
    # ---- the whole PairFormerBlock in fp32, wall clock; informative
    pf32 = of3pair.PairFormerBlock(C_S, 128, C_HEAD_S, PAIR_BIAS_HEADS, 128, 32, 4, "swiglu", TRANSITION_N, 0.25, False, 1e9)
    pf32.load_state_dict(pf.state_dict())
    pf32 = pf32.to(dev).float().eval()
    s32 = s_pf.float()
    pf32(s32, z32, sm, m32)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(fp32_reps):
        pf32(s32, z32, sm, m32)
    torch.cuda.synchronize()
    fp32_pairformer_block_ms = (time.perf_counter() - t0) * 1e3 / fp32_reps

    # ---- one block of the template pair stack at its own shape (4 templates, N = 512, c_t = 64, 4 x 16), both
    # precisions, wall clock; informative
    template_block_ms = {}
    t_gen = torch.Generator().manual_seed(3)
    t_params = dict(orc.make_block_params(30, 64, 64, 16, 4))
    t_params.update({"pair_transition." + k_: v for k_, v in orc.make_transition_params(t_gen, 64, 2).items()})
    t_host = orc.make_pair_input(3, (4,), 512, 64)
    t_mask = orc.tail_padding_mask((4,), 512, torch.tensor([0, 20, 51, 102])).to(dev)
    for name, dt in (("bf16", bf), ("fp32", torch.float32)):
        tb_ = of3pair.PairBlock(64, 64, 16, 4, "swiglu", 2, 0.0, False, 1e9)
        tb_.load_state_dict(t_params, strict=True)
        tb_ = tb_.to(dev).to(dt).eval()
        t_in = t_host.to(dev).to(dt)
        tb_(t_in, t_mask)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(fp32_reps):
            tb_(t_in, t_mask)
        torch.cuda.synchronize()
        template_block_ms[name] = round((time.perf_counter() - t0) * 1e3 / fp32_reps, 3)
        del tb_, t_in
    return fp32_pairformer_block_ms, template_block_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--n", type=int, default=768, help="N_token (768 = the headline configuration)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the fp32 PairFormerBlock and the template-block legs (profiles of the headline workload)")
    ap.add_argument("--contract-variant", type=int, default=0)
    ap.add_argument("--configs", default="2,4,5",
                    help="which of the other benchmark configurations (2, 4, 5) to time as well; '' for none")
    ap.add_argument("--configs-only", action="store_true",
                    help="time only the configurations named by --configs (kernel traces of one configuration); prints "
                         "their figures, no headline line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build is single-GPU (one pair-stack block on one MI355X); run with --gpus 1")

    import torch

    from of3pair import _lib
    from of3pair import build as of3_build

    if not of3_build.is_built():
        of3_build.build()
    import of3pair
    from oracle import pairstack_oracle as orc

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, N, C, CH, H, D = 1, args.n, 128, 128, 4, 32

    if args.configs_only:
        which = [int(c) for c in args.configs.split(",") if c]
        print(json.dumps({"configs": other_configs(of3pair, _lib.load(), _lib, orc, torch, dev, which)}))
        return

    params = {k: orc.round_bf16(v) for k, v in orc.make_block_params(0, C, CH, D, H).items()}
    block = of3pair.PairStack(C, CH, D, H)
    block.load_state_dict(params)
    block = block.to(dev).to(torch.bfloat16).eval()
    z_host = orc.round_bf16(orc.make_pair_input(1, (B,), N, C))
    z = z_host.to(dev).to(torch.bfloat16)
    mask = torch.ones(B, N, N, device=dev)

    # one plain device copy of known size (CAL_BYTES read + CAL_BYTES written): a counter
    # profile of this command then holds its own calibration kernel for FETCH_SIZE/WRITE_SIZE
    cal_src = torch.ones(CAL_BYTES // 4, dtype=torch.float32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    # ---- whole block, inputs resident, the same input in every step
    def step():
        return block(z, mask, inplace_safe=False)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # the same K steps once more with one event pair per step: spread of the step time
    step_marks = []
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        step_marks.append((e0, e1))
    torch.cuda.synchronize()
    step_ms = sorted(e0.elapsed_time(e1) for e0, e1 in step_marks)
    step_ms_median, step_ms_min = step_ms[len(step_ms) // 2], step_ms[0]

    # and in place (the z of step k is the output of step k-1), for comparison
    z_ip = z.clone()
    block(z_ip, mask, inplace_safe=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        block(z_ip, mask, inplace_safe=True)
    torch.cuda.synchronize()
    inplace_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    del z_ip

    # ---- per-kernel durations: the same block issued kernel by kernel through the stage
    # entry points of the C ABI, every launch bracketed by its own pair of events on the
    # launch stream, so that each kernel is timed where it runs in the block (inputs left in
    # the caches by its producer, clocks as in the block) and not in a back-to-back loop
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    bf = torch.bfloat16
    zz = z_host.to(dev).to(bf)
    dp = {k: v.to(dev).to(bf).contiguous() for k, v in params.items()}
    block_launches, keep = block_stage_launches(lib, _lib, torch, dp, zz, mask, (B, N, C, CH, H, D), args.contract_variant)
    z_fwd, m_fwd = keep[-4], keep[-2]
    P = lambda t: t.data_ptr()  # noqa: E731

    def ck(st):
        _lib.check(st, "bench stage")

    tgen = torch.Generator().manual_seed(7)
    tp = {k_: v.to(dev).to(bf).contiguous() for k_, v in orc.make_transition_params(tgen, C, TRANSITION_N).items()}
    transition = [("pair_transition", lambda: ck(lib.of3_transition_fwd(
        P(zz), z_fwd, P(mask), m_fwd, P(tp["layer_norm.weight"]), P(tp["layer_norm.bias"]),
        P(tp["swiglu.linear_a.weight"]), P(tp["swiglu.linear_b.weight"]), P(tp["linear_out.weight"]), P(zz),
        B, N, C, TRANSITION_N * C, 1, _lib.OF3_DTYPE_BF16, s)))]
    bp = {k_: v.to(dev).to(bf).contiguous() for k_, v in orc.make_pair_bias_params(tgen, C, PAIR_BIAS_HEADS).items()}
    bias_out = torch.empty(B, PAIR_BIAS_HEADS, N, N, dtype=bf, device=dev)
    pair_bias = [("pair_bias_proj", lambda: ck(lib.of3_pair_bias_fwd(
        P(zz), z_fwd, P(bp["layer_norm_z.weight"]), P(bp["layer_norm_z.bias"]), P(bp["linear_z.weight"]),
        P(bias_out), B, N, C, PAIR_BIAS_HEADS, _lib.OF3_DTYPE_BF16, s)))]
    ttp = {k_: v.to(dev).to(bf).contiguous() for k_, v in orc.make_template_tail_params(tgen, C_T, C).items()}
    t_in = torch.randn(B, TEMPLATES, N, N, C_T, device=dev).to(bf)
    t_out = torch.empty(B, N, N, C, dtype=bf, device=dev)
    template_tail = [("template_tail", lambda: ck(lib.of3_template_tail_fwd(
        P(t_in), P(ttp["template_pair_stack.layer_norm.weight"]), P(ttp["template_pair_stack.layer_norm.bias"]),
        P(ttp["linear_t.weight"]), P(t_out), B, TEMPLATES, N * N, C_T, C, 1, _lib.OF3_DTYPE_BF16, s)))]
    sp = {k_: v.to(dev).to(bf).contiguous()
          for k_, v in orc.make_attention_pair_bias_params(tgen, C_S, C, C_HEAD_S, PAIR_BIAS_HEADS).items()}
    s_in = torch.randn(B, N, C_S, device=dev).to(bf)
    s_out = torch.empty_like(s_in)
    s_ws = torch.empty(int(lib.of3_attn_pair_bias_workspace_bytes(B, N, C_S, PAIR_BIAS_HEADS, C_HEAD_S)),
                       dtype=torch.uint8, device=dev)
    attn_pair_bias = [("attn_pair_bias", lambda: ck(lib.of3_attn_pair_bias_fwd(
        P(s_in), P(bias_out), None, P(sp["layer_norm_a.weight"]), P(sp["layer_norm_a.bias"]),
        P(sp["mha.linear_q.weight"]), P(sp["mha.linear_q.bias"]), P(sp["mha.linear_k.weight"]),
        P(sp["mha.linear_v.weight"]), P(sp["mha.linear_g.weight"]), P(sp["mha.linear_o.weight"]), P(s_out),
        B, N, C_S, PAIR_BIAS_HEADS, C_HEAD_S, 1e9, 0, P(s_ws), s_ws.numel(), _lib.OF3_DTYPE_BF16, s)))]
    stp = {k_: v.to(dev).to(bf).contiguous() for k_, v in orc.make_transition_params(tgen, C_S, TRANSITION_N).items()}
    st_ws = torch.empty(int(lib.of3_transition_rows_workspace_bytes(B * N, C_S, TRANSITION_N * C_S)),
                        dtype=torch.uint8, device=dev)
    single_transition = [("single_transition", lambda: ck(lib.of3_transition_rows_fwd(
        P(s_in), None, P(stp["layer_norm.weight"]), P(stp["layer_norm.bias"]), P(stp["swiglu.linear_a.weight"]),
        P(stp["swiglu.linear_b.weight"]), P(stp["linear_out.weight"]), P(s_out), B * N, C_S, TRANSITION_N * C_S, 0,
        P(st_ws), st_ws.numel(), _lib.OF3_DTYPE_BF16, s)))]
    launches = (block_launches + transition + pair_bias + attn_pair_bias + single_transition + template_tail)
    durations = time_launches(torch, launches, args.steps, args.warmup)
    kernels = kernel_figures(durations, kernel_model(B, N, C, CH, H, D))
    dom = kernels["trimul_contract"]
    roofline = {"kernel": "trimul_contract", "bound": "mfma", "achieved": dom["achieved"], "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": dom["frac"],
                "traffic": MEASURED_TRAFFIC.get((N, args.contract_variant or int(lib.of3_trimul_contract_variant(B, N, CH))))}

    # ---- a whole PairFormerBlock through the module interface (pair stack, pair transition, pair
    # bias, attention over s, single transition), wall clock; informative, not part of `value`
    import of3pair
    pf = of3pair.PairFormerBlock(C_S, C, C_HEAD_S, PAIR_BIAS_HEADS, CH, D, H, "swiglu", TRANSITION_N, 0.25, False, 1e9)
    pf.load_state_dict({k_: v for k_, v in orc.make_pairformer_block_params(0, C_S, C, CH, D, H, C_HEAD_S,
                                                                             PAIR_BIAS_HEADS, TRANSITION_N).items()})
    pf = pf.to(dev).to(bf).eval()
    s_pf, z_pf = torch.randn(B, N, C_S, device=dev).to(bf), z_host.to(dev).to(bf)
    sm, pm = torch.ones(B, N, device=dev), torch.ones(B, N, N, device=dev)
    for _ in range(2):
        pf(s_pf, z_pf, sm, pm)  # not in place: every repetition sees the same input
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        pf(s_pf, z_pf, sm, pm)
    torch.cuda.synchronize()
    pairformer_block_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- the same pair-stack block in fp32 through the module interface, wall clock; informative
    ps32 = of3pair.PairStack(C, CH, D, H)
    ps32.load_state_dict(params, strict=True)
    ps32 = ps32.to(dev).eval()
    z32, m32 = z_host.to(dev), torch.ones(B, N, N, device=dev)
    ps32(z32, m32)
    torch.cuda.synchronize()
    fp32_reps = max(1, min(5, args.steps))
    t0 = time.perf_counter()
    for _ in range(fp32_reps):
        ps32(z32, m32)
    torch.cuda.synchronize()
    fp32_block_ms = (time.perf_counter() - t0) * 1e3 / fp32_reps

    fp32_pairformer_block_ms, template_block_ms = None, None
    if not args.no_extras:
        fp32_pairformer_block_ms, template_block_ms = extra_legs(of3pair, orc, pf, s_pf, z32, sm, m32, fp32_reps, dev)
    del pf, ps32, z32, m32, launches, block_launches, keep
    torch.cuda.empty_cache()
    which = [int(c) for c in args.configs.split(",") if c]
    configs = other_configs(of3pair, lib, _lib, orc, torch, dev, which) if which else None

    # ---- CPU baseline: the oracle on the host cores, one block of the same workload; one warm-up
    # run (thread pool, allocator), then the median of three
    cpu = None
    if not args.no_cpu:
        torch.set_num_threads(os.cpu_count() or 1)
        mask_h = torch.ones(B, N, N)
        runs = []
        for rep in range(4):
            t0 = time.perf_counter()
            with torch.no_grad():
                orc.pair_stack_block(z_host, mask_h, params, H, row_chunk=32)
            if rep > 0:
                runs.append((time.perf_counter() - t0) * 1e3)
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as f:
                for ln in f:
                    if ln.startswith("model name"):
                        cpu_model = ln.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        cpu = {"value": round(sorted(runs)[1], 1), "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
               "cpu": cpu_model, "runs_ms": [round(r, 1) for r in runs],
               "sample": "1 block forward, fp32, N=%d, same weights and input (tri-attn in 32-row chunks); "
                         "median of 3 after one warm-up run" % N}

    line = {
        "metric": METRIC, "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "step_ms_median": round(step_ms_median, 4),
        "step_ms_min": round(step_ms_min, 4), "inplace_ms_per_step": round(inplace_ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "pair-stack block (trimul out+in, tri-attn start+end, residuals), B=1, N_token=%d, "
                               "c_z=128, c_hidden_mul=128, 4 heads x 32, all-ones mask" % N},
        "roofline": roofline, "kernels": kernels, "cpu_baseline": cpu,
        "pairformer_block_ms": round(pairformer_block_ms, 4), "fp32_block_ms": round(fp32_block_ms, 3),
        "fp32_pairformer_block_ms": None if fp32_pairformer_block_ms is None else round(fp32_pairformer_block_ms, 3),
        "template_block_ms": template_block_ms, "configs": configs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
