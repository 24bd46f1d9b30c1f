#!/usr/bin/env python3
"""Benchmark of the dynamic-mask attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all] [--legs a,b,...] [--no-cpu]

A "step" is one forward pass of `flash_sparse_attn_func` over one synthetic batch of the headline
configuration: B=1, Lq=Lk=8192, H=32, Hkv=8 (GQA 4:1), d=128, bf16, bias [B,Hkv,1,Lk] ~ N(0,1),
keep-mask = per-row top-2048 keys by bias intersected with causal, scale 1/sqrt(128).
Prints ONE JSON line.  `value` is the forward's effective TFLOP/s counting only executed tiles on
the canonical 64x64 tile grid (a tile is executed iff it holds at least one mask-and-causal-visible
element); forward+backward, the other benchmark configurations (`configs`: cfg3 and the decode shape cfg5
against HBM, cfg4 against the matrix pipe, each with its own roofline block), the forward's runtime against the
window W (`w_sweep_fwd`, with the fitted line), the roofline of the dominant kernel and a CPU baseline on the host
cores ride along in the same line.

Inputs are resident in HBM before the timed region starts; timing uses HIP events on the stream the
kernels are launched on (torch's current stream).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-dmattn_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# HBM bytes per launch of the forward kernel on the headline workload come from two rocprofv3 --pmc runs of this
# script (FETCH_SIZE, WRITE_SIZE; each scaled by what the counter reads for a 256 MiB device copy, see --calib-copy).
# `python bench.py --summarise-pmc <fetch csv> <write csv>` turns the two counter files into TRAFFIC_FILE, which is
# tracked; a normal run reports what that file says (null when it is missing).  --traffic-bytes overrides it.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "fwd_colmask_cfg2_hbm_traffic.txt")


def read_traffic(compacted):
    """HBM bytes per launch of the forward kernel (compacted or tile-skipping variant) from TRAFFIC_FILE, or None."""
    key = "compacted_bytes" if compacted else "tile_skip_bytes"
    try:
        for line in open(TRAFFIC_FILE):
            if line.startswith(key + " ="):
                return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def summarise_pmc(fetch_csv, write_csv):
    """Reads the counter_collection CSVs of the two --pmc passes (FETCH_SIZE, then WRITE_SIZE; both with --calib-copy)
    and writes TRAFFIC_FILE: per forward kernel variant, read + written HBM bytes per launch, each counter scaled by
    what it reads for the 256 MiB copy."""
    import csv
    import re

    def per_kernel(path, counter):
        """mean per dispatch of every kernel, and the largest value among the runtime's copy kernel dispatches: the
        process makes other, small device copies too; the 256 MiB calibration copy is the largest of them"""
        acc = {}
        for row in csv.DictReader(open(path)):
            if row.get("Counter_Name") != counter:
                continue
            name = row["Kernel_Name"]
            acc.setdefault(name, []).append(float(row["Counter_Value"]))
        copies = [max(v) for k, v in acc.items() if "copyBuffer" in k]
        return {k: sum(v) / len(v) for k, v in acc.items()}, max(copies)

    (fetch, f_copy), (write, w_copy) = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    copy_kib = 256.0 * 1024
    f_scale = copy_kib / f_copy
    w_scale = copy_kib / w_copy
    lines = ["# HBM traffic per launch of fdma::fwd_colmask_kernel on bench.py's headline workload (cfg2), written by",
             "# `python bench.py --summarise-pmc`; FETCH_SIZE / WRITE_SIZE are KiB per dispatch, scaled by the factors below",
             "fetch_scale = %.4f" % f_scale, "write_scale = %.4f" % w_scale]
    for key, cmp_flag in (("compacted_bytes", "true"), ("tile_skip_bytes", "false")):
        # (the compacted forward of the headline workload is the streaming kernel; its pre-pass is a launch of its own)
        pat = re.compile(r"fwd_stream_kernel<" if cmp_flag == "true" else r"fwd_colmask_kernel<.*128.*, false>")
        fk = [v for k, v in fetch.items() if pat.search(k)]
        wk = [v for k, v in write.items() if pat.search(k)]
        if fk and wk:
            lines.append("%s = %.0f   (read %.1f MiB + written %.1f MiB)" % (
                key, (fk[0] * f_scale + wk[0] * w_scale) * 1024, fk[0] * f_scale / 1024, wk[0] * w_scale / 1024))
    open(TRAFFIC_FILE, "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))

CONFIGS = {
    # name: B, Lq, Lk, H, Hk, D, bias shape, window, causal, passes
    "cfg1": dict(B=1, Lq=256, Lk=256, H=2, Hk=1, D=64, bias=(1, 1, 1, 256), W=128, causal=True, bwd=True, scale=0.125),
    "cfg2": dict(B=1, Lq=8192, Lk=8192, H=32, Hk=8, D=128, bias=(1, 8, 1, 8192), W=2048, causal=True, bwd=True, scale=None),
    "cfg3": dict(B=2, Lq=4096, Lk=4096, H=16, Hk=16, D=64, bias=(2, 16, 4096, 4096), W=1024, causal=True, bwd=True, scale=None),
    "cfg4": dict(B=1, Lq=32768, Lk=32768, H=16, Hk=4, D=128, bias=(1, 4, 1, 32768), W=1024, causal=True, bwd=True, scale=None),
    "cfg5": dict(B=8, Lq=1, Lk=65536, H=32, Hk=8, D=128, bias=(8, 8, 1, 65536), W=2048, causal=False, bwd=False, scale=None),
}


def make_case(c, device, seed=0):
    """Synthetic inputs.  The mask has the bias's shape (top-W per row); the causal intersection is
    applied by is_causal=True, which is the identical keep-set."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    dt = torch.bfloat16
    q = torch.randn(c["B"], c["Lq"], c["H"], c["D"], generator=g).to(dt).to(device)
    k = torch.randn(c["B"], c["Lk"], c["Hk"], c["D"], generator=g).to(dt).to(device)
    v = torch.randn(c["B"], c["Lk"], c["Hk"], c["D"], generator=g).to(dt).to(device)
    if c["bias"][2] == 1:
        bias = torch.randn(*c["bias"], generator=g).to(dt).to(device)
    else:  # the per-query bias of cfg3 is 1 GiB: draw it on the device
        gd = torch.Generator(device=device).manual_seed(seed)
        bias = torch.randn(*c["bias"], generator=gd, device=device, dtype=torch.float32).to(dt)
    idx = bias.float().topk(min(c["W"], c["Lk"]), dim=-1).indices
    mask = torch.zeros(bias.shape, dtype=torch.bool, device=device).scatter_(-1, idx, True)
    return q, k, v, mask, bias


def count_tiles(mask, Lq, Lk, causal, H, tile=64):
    """Canonical 64x64 tile statistics from the actual mask: (executed tiles, causal tiles, nnz)
    summed over batch and query heads."""
    Bm, Hm, Rm, _ = mask.shape
    shift = Lk - Lq
    nq, nk = (Lq + tile - 1) // tile, (Lk + tile - 1) // tile
    dev = mask.device
    last_row = torch.clamp(torch.arange(nq, device=dev) * tile + tile - 1, max=Lq - 1)  # most permissive row
    kblock_lo = torch.arange(nk, device=dev) * tile
    causal_tile = (kblock_lo[None, :] <= last_row[:, None] + shift) if causal else torch.ones(nq, nk, dtype=torch.bool, device=dev)
    rep = H // Hm
    if Rm == 1:
        m = mask[:, :, 0, :Lk]
        pad = nk * tile - Lk
        mp = torch.nn.functional.pad(m, (0, pad)).view(Bm, Hm, nk, tile)
        cols = torch.arange(nk * tile, device=dev).view(nk, tile)
        big = torch.iinfo(torch.int64).max
        first_kept = torch.where(mp, cols, torch.full_like(cols, big)).min(-1).values  # (Bm,Hm,nk)
        if causal:
            ex = first_kept[:, :, None, :] <= last_row[None, None, :, None] + shift
            executed = int(ex.sum().item()) * rep
        else:
            executed = int((first_kept < big).sum().item()) * nq * rep
        if causal:
            rows = torch.arange(Lq, device=dev)
            csum = torch.cumsum(m.to(torch.int64), -1)
            lim = torch.clamp(rows + shift, max=Lk - 1)
            nnz = int(torch.where(lim >= 0, csum[..., torch.clamp(lim, min=0)], torch.zeros((), dtype=torch.int64, device=dev)).sum().item()) * rep
        else:
            nnz = int(m.sum().item()) * Lq * rep
    else:
        executed, nnz = 0, 0
        cm = None
        if causal:
            i = torch.arange(Lq, device=dev)[:, None]
            j = torch.arange(Lk, device=dev)[None, :]
            cm = j <= i + shift
        for b in range(Bm):
            for h in range(Hm):
                m = mask[b, h, :, :Lk]
                if cm is not None:
                    m = m & cm
                nnz += int(m.sum().item())
                mp = torch.nn.functional.pad(m, (0, nk * tile - Lk, 0, nq * tile - Lq))
                executed += int(mp.view(nq, tile, nk, tile).any(3).any(1).sum().item())
        executed *= rep
        nnz *= rep
    Bfull = mask.shape[0]
    return executed, int(causal_tile.sum().item()) * H * Bfull, nnz


def compaction_applies(mask, c):
    """Mirror of the library's rule for taking the column-compaction path (query-broadcast keep-mask with
    1 or Hkv heads, a problem large enough for the pre-pass to pay, not switched off)."""
    from flash_sparse_attn import _cabi
    mode = {_cabi.COMPACT_NEVER: "0", _cabi.COMPACT_ALWAYS: "2"}.get(_cabi.get_compact_mode(), "1")
    form_ok = mask.shape[2] == 1 and mask.shape[1] in (1, c["Hk"]) and c["Lq"] >= 2
    pays = c["Lq"] >= 128 and c["Lk"] >= 128 and c["Lq"] * (c["H"] // c["Hk"]) * c["Lk"] >= 1 << 21
    return mode != "0" and form_ok and (mode == "2" or pays)


def count_compacted_tiles(mask, Lq, Lk, causal, H, tile=64):
    """64x64 tiles the compacted kernels execute: per (batch, mask head) the kept columns are packed to the
    front, and a 64-row query block runs over ceil(visible / 64) tiles, visible = kept columns at or below
    the causal limit of the block's last row.  Summed over batch and query heads."""
    Bm, Hm, _, _ = mask.shape
    dev = mask.device
    m = mask[:, :, 0, :Lk]
    csum = torch.cumsum(m.to(torch.int64), -1)
    nq = (Lq + tile - 1) // tile
    if causal:
        last_row = torch.clamp(torch.arange(nq, device=dev) * tile + tile - 1, max=Lq - 1)
        lim = last_row + (Lk - Lq)
        vis = torch.where(lim >= 0, csum[..., torch.clamp(lim, 0, Lk - 1)], torch.zeros((), dtype=torch.int64, device=dev))
    else:
        vis = csum[..., -1:].expand(Bm, Hm, nq)
    return int(((vis + tile - 1) // tile).sum().item()) * (H // Hm)


RAMP_SECONDS = 0.25  # busy time before the warm-up steps: an idle MI355X takes that long to reach its running clocks


def time_gpu(fn, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` timed ones between two events on the current stream.  Before
    both, the same step runs for RAMP_SECONDS so that a cold device (power state, clocks) does not dominate a
    timed region of a few milliseconds.  The first call (library and code-object loading on the host) is made
    before the ramp clock starts: it can take longer than RAMP_SECONDS with the device idle."""
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < RAMP_SECONDS:
        fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def run_config(name, steps, warmup, device, compact=True, backward=True, zero_inputs=False):
    from flash_sparse_attn import _cabi, flash_sparse_attn_func

    _cabi.set_compact_mode(_cabi.COMPACT_AUTO if compact else _cabi.COMPACT_NEVER)  # the compact_mode field of every call
    c = CONFIGS[name]
    q, k, v, mask, bias = make_case(c, device)
    if zero_inputs:  # same mask, same tiles, same instruction stream; operands that do not toggle the data paths
        q, k, v, bias = [torch.zeros_like(t) for t in (q, k, v, bias)]
    scale = c["scale"]
    res = {"name": name, "mask_form": "[B,Hm,%s,Lk] bool + is_causal" % ("1" if mask.shape[2] == 1 else "Lq")}
    with torch.no_grad():
        ms_fwd = time_gpu(lambda: flash_sparse_attn_func(q, k, v, mask, bias, scale, c["causal"]), steps, warmup)
    res["ms_fwd"] = ms_fwd
    if c["Lq"] > 1:
        n_exec, n_causal, nnz = count_tiles(mask, c["Lq"], c["Lk"], c["causal"], c["H"])
        res.update(n_exec=n_exec, n_causal_tiles=n_causal, tile_occupancy=n_exec / max(1, n_causal), nnz=nnz)
        res["compacted"] = compaction_applies(mask, c)
        if res["compacted"]:
            # the kernels run on the compacted key axis: their executed tiles are counted there; the tile
            # count of the original layout (what a tile-skipping kernel would execute) is kept beside it
            res["n_exec_original_layout"] = n_exec
            res["tflops_fwd_original_layout_tiles"] = 4.0 * 64 * 64 * c["D"] * n_exec / ms_fwd / 1e9
            n_exec = count_compacted_tiles(mask, c["Lq"], c["Lk"], c["causal"], c["H"])
            res["n_exec"] = n_exec
        fl_fwd = 4.0 * 64 * 64 * c["D"] * n_exec
        res["tflops_fwd"] = fl_fwd / ms_fwd / 1e9
        res["tflops_fwd_elementwise"] = 4.0 * c["D"] * nnz / ms_fwd / 1e9
    else:
        kept = int(mask.sum().item())  # per (b, mask head); all heads of a group share the rows
        rows = kept * (c["Hk"] // mask.shape[1] if mask.shape[1] <= c["Hk"] else 1)
        kv_bytes = 2.0 * rows * c["D"] * 2
        side = mask.numel() + bias.numel() * 2 + q.numel() * 2 * 2
        res.update(kept_rows=rows, touched_bytes=kv_bytes + side, hbm_gbs=(kv_bytes + side) / ms_fwd / 1e6,
                   hbm_gbs_tile64=None)
        m = mask[:, :, 0, :]
        blocks = int(m.view(m.shape[0], m.shape[1], -1, 64).any(-1).sum().item())
        res["tile64_bytes"] = 2.0 * blocks * 64 * c["D"] * 2 + side
        res["hbm_gbs_tile64"] = res["tile64_bytes"] / ms_fwd / 1e6
    if c["bwd"] and backward:
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
        bg = bias.clone().requires_grad_(True)

        dout = torch.ones_like(q)  # upstream gradient, resident like the other inputs

        def step():
            qg.grad = kg.grad = vg.grad = bg.grad = None  # (first: no accumulation pass over a gradient left from the step before)
            out = flash_sparse_attn_func(qg, kg, vg, mask, bg, scale, c["causal"])
            out.backward(dout)

        ms_fb = time_gpu(step, max(2, steps // 2), max(1, warmup // 2))
        res["ms_fwd_bwd"] = ms_fb
        res["tflops_fwd_bwd"] = 14.0 * 64 * 64 * c["D"] * res["n_exec"] / ms_fb / 1e9
    return res


def run_mfma_probe():
    """What rate of bf16 MFMA 32x32x16 the device sustains on its own (flash-dmattn_amd/csrc/fdma_probe.hip, built
    next to the library): 256 workgroups of 8 waves issuing nothing but MFMAs from registers, the same with one LDS
    fragment read per MFMA, and with the forward kernel's vector work per MFMA on top -- on constant and on random
    operands.  The published peak assumes 2.4 GHz; real operands make the device run slower, so `roofline.frac`
    (always against the published peak) is to be read next to these.  Returns None when the probe is not built."""
    import ctypes

    path = os.path.join(ROOT, "flash-dmattn_amd", "lib", "libfdma_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.fdma_probe_mfma_tflops.restype = ctypes.c_double
    lib.fdma_probe_mfma_tflops.argtypes = [ctypes.c_int, ctypes.c_int]
    names = ("registers_only", "lds_fragment_per_mfma", "lds_fragment_and_softmax_valu_per_mfma")
    out = {"unit": "TFLOP/s", "note": "bf16 MFMA 32x32x16 alone, 256 workgroups x 8 waves; the softmax mix is 2 exp2 + 1 "
                                      "conversion + 2 additions per MFMA"}
    for mode, name in enumerate(names):
        out[name] = {"constant_operands": lib.fdma_probe_mfma_tflops(mode, 0), "random_operands": lib.fdma_probe_mfma_tflops(mode, 1)}
    return out


def run_hbm_probe():
    """What rate of bytes the device delivers to a kernel that only reads 256-byte rows (a K or V row at head dim 128),
    one launch each, launch ramp included: a stream of 1 GiB, 1 GiB of rows at scattered positions, and cfg5's volume
    (2 x 131072 kept rows = 67 MB) at scattered positions of a 2 GiB buffer -- what the gather of a decode call looks
    like to the memory, without the mask, the lists, the arithmetic and the merge.  The HBM roofline fractions (always
    against the published 8 TB/s) are to be read next to these.  None when the probe is not built."""
    import ctypes

    path = os.path.join(ROOT, "flash-dmattn_amd", "lib", "libfdma_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    if not hasattr(lib, "fdma_probe_read_gbs"):
        return None
    lib.fdma_probe_read_gbs.restype = ctypes.c_double
    lib.fdma_probe_read_gbs.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_int]
    out = {"unit": "GB/s", "row_bytes": 256,
           "stream_1GiB": lib.fdma_probe_read_gbs(1 << 22, 0, 1024),
           "scattered_rows_1GiB": lib.fdma_probe_read_gbs(1 << 22, 1, 2048),
           "scattered_rows_cfg5_volume_67MB": lib.fdma_probe_read_gbs(2 * 131072, 1, 2048),
           "note": "read-only kernels, best of five launches each; scattered = hashed row positions in a 2 GiB buffer"}
    if hasattr(lib, "fdma_probe_tile_walk_gbs"):
        # cfg3's access pattern alone: 128-row workgroups walking a [4096, 4096] bias and mask 64 columns at a time, at the
        # general forward kernel's occupancy and depth (two workgroups of four waves per CU, one step in flight)
        lib.fdma_probe_tile_walk_gbs.restype = ctypes.c_double
        lib.fdma_probe_tile_walk_gbs.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
        out["tile_walk_mask_and_bias_cfg3_pattern"] = lib.fdma_probe_tile_walk_gbs(1, 1, 64)
        out["tile_walk_mask_and_bias_4_workgroups_per_cu"] = lib.fdma_probe_tile_walk_gbs(1, 1, 0)
        out["tile_walk_bias_only"] = lib.fdma_probe_tile_walk_gbs(0, 1, 64)
    return out


def config_roofline(name, r):
    """Roofline block of one of the secondary configurations (the headline's is built in main()): the bound of
    the configuration (matrix pipe for the column-mask shapes, HBM for per-query bias and for decode), the algorithmic
    work per call and what the measured call time makes of it.  Durations are whole operator calls (all launches of the call), timed with events on the
    launch stream."""
    c = CONFIGS[name]
    if c["Lq"] == 1:  # decode: HBM, touched K / V rows + side inputs
        blk = {"bound": "hbm", "unit": "GB/s", "peak": PEAK_HBM_GBS, "bytes_per_call": r["touched_bytes"],
               "bytes_model": "2 (K, V) * kept rows * d * 2 B + mask bytes + bias + q / out; kept rows counted from the mask",
               "achieved": r["hbm_gbs"], "frac": r["hbm_gbs"] / PEAK_HBM_GBS, "duration_ms": r["ms_fwd"],
               "kernel": "fdma::decode_kernel (the last workgroup of a (batch entry, kv head) merges the splits), whole operator call"}
        if "ms_fwd_c_abi" in r:
            gbs = r["touched_bytes"] / r["ms_fwd_c_abi"] / 1e6
            blk["c_abi_call"] = {"duration_ms": r["ms_fwd_c_abi"], "achieved": gbs, "frac": gbs / PEAK_HBM_GBS}
        return blk
    if r["mask_form"].endswith("Lq,Lk] bool + is_causal"):  # per-query mask and bias: HBM
        B, H, Lq, Lk, D = c["B"], c["H"], c["Lq"], c["Lk"], c["D"]
        n_causal = r["n_causal_tiles"]
        q_bytes, kv_bytes, lse_bytes = 2.0 * B * Lq * H * D, 2.0 * B * Lk * c["Hk"] * D, 4.0 * B * H * Lq
        tiles = n_causal * 64 * 64 * 1.0 + r["n_exec"] * 64 * 64 * 2.0  # mask of every causal tile, bias of every executed one
        fwd = tiles + 2 * q_bytes + 2 * kv_bytes + lse_bytes            # q, out, k, v
        # backward, algorithmic minimum: the tiles once more, every dBias element written once (zeros included),
        # q / out / dout read and dq written, k / v read and dk / dv written
        bwd = tiles + 2.0 * B * H * Lq * Lk + 4 * q_bytes + 4 * kv_bytes + lse_bytes
        blk = {"bound": "hbm", "unit": "GB/s", "peak": PEAK_HBM_GBS, "bytes_per_call": fwd,
               "bytes_model": "forward: mask bytes of every causal 64x64 tile + bias of every executed tile + q, k, v, out, lse; "
                              "forward + backward adds the same tiles once more, the full dBias write, dout and the gradients "
                              "(measured traffic is higher: the dQ kernel reads the written dS tiles back, see profiles/)",
               "achieved": fwd / r["ms_fwd"] / 1e6, "frac": fwd / r["ms_fwd"] / 1e6 / PEAK_HBM_GBS, "duration_ms": r["ms_fwd"],
               "kernel": "fdma::fwd_kernel (per-query mask / bias), whole operator call"}
        if "ms_fwd_bwd" in r:
            tot = fwd + bwd
            blk["fwd_bwd"] = {"bytes_per_call": tot, "duration_ms": r["ms_fwd_bwd"], "achieved": tot / r["ms_fwd_bwd"] / 1e6,
                              "frac": tot / r["ms_fwd_bwd"] / 1e6 / PEAK_HBM_GBS,
                              "kernels": "fwd_kernel, bwd_dot_kernel, bwd_dkdv_kernel, bwd_dq_ds_kernel (dQ from the dS tiles that dK/dV wrote as dBias)"}
        return blk
    flops = 4.0 * 64 * 64 * c["D"] * r["n_exec"]
    blk = {"bound": "mfma", "unit": "TFLOP/s", "peak": PEAK_BF16_TFLOPS, "flops_per_call": flops,
           "flops_model": "4*64*64*d per executed 64x64 tile (compacted key axis when column_compaction), 14*... forward + backward",
           "column_compaction": bool(r.get("compacted")), "n_exec_tiles": r["n_exec"],
           "achieved": r["tflops_fwd"], "frac": r["tflops_fwd"] / PEAK_BF16_TFLOPS, "duration_ms": r["ms_fwd"],
           "kernel": "fdma::fwd_stream_kernel with its pre-pass (compact_scan_image_kernel), whole operator call" if r.get("compacted") else "fdma::fwd_colmask_kernel (tile skipping), whole operator call"}
    if "ms_fwd_bwd" in r:
        blk["fwd_bwd"] = {"flops_per_call": 3.5 * flops, "duration_ms": r["ms_fwd_bwd"], "achieved": r["tflops_fwd_bwd"],
                          "frac": r["tflops_fwd_bwd"] / PEAK_BF16_TFLOPS}
    return blk


def time_decode_c_abi(name, steps, warmup, device):
    """The decode configuration through the C ABI alone: one prepared argument block, fdma_fwd called back to back on
    torch's current stream (what a serving loop written against include/fdma.h pays per call)."""
    from flash_sparse_attn import _cabi

    c = CONFIGS[name]
    q, k, v, mask, bias = make_case(c, device)
    out = torch.empty_like(q)
    lse = torch.empty((c["B"], c["H"], c["Lq"]), dtype=torch.float32, device=device)
    args = _cabi.FwdArgs()
    _cabi.fill_fwd(args, q, k, v, mask, bias, out, lse, c["D"] ** -0.5, c["causal"], 0.0, None, None)
    nbytes = _cabi.lib.fdma_fwd_workspace_bytes(args)
    ws = torch.empty(max(1, nbytes), dtype=torch.uint8, device=device)
    if nbytes:
        args.workspace, args.workspace_bytes = ws.data_ptr(), nbytes
    cbytes = _cabi.lib.fdma_fwd_counter_bytes(args)  # arrival counters: the splits are merged by the decode launch itself
    counters = torch.zeros(max(1, cbytes // 4), dtype=torch.int32, device=device)
    if cbytes:
        args.counters, args.counters_bytes = counters.data_ptr(), cbytes
    stream = _cabi.current_stream(device)

    def call():
        _cabi.check(_cabi.lib.fdma_fwd(args, stream))

    return time_gpu(call, steps, warmup)


def run_w_sweep_fwd(steps, warmup, device):
    """Forward time against the window W at L = 8192 (H=32, Hkv=8, d=128, bias [1,8,1,L], mask = top-W of the bias,
    causal), default path and tile skipping alone, with a least-squares line ms = a + b * W per path (the reference's
    claim: runtime grows linearly with the window, README.md:181-191, benchmarks/forward_performance.py:661-718)."""
    rows = []
    for W in (256, 512, 1024, 2048, 4096, 8192):
        CONFIGS["_sweep"] = dict(B=1, Lq=8192, Lk=8192, H=32, Hk=8, D=128, bias=(1, 8, 1, 8192), W=W, causal=True, bwd=False, scale=None)
        row = {"W": W}
        for compact, tag in ((True, "default"), (False, "tile_skip")):
            r = run_config("_sweep", steps, warmup, device, compact, backward=False)
            row["ms_fwd_" + tag] = r["ms_fwd"]
            row["n_exec_" + tag] = r["n_exec"]
            row["tflops_fwd_" + tag] = r["tflops_fwd"]
        rows.append(row)
    del CONFIGS["_sweep"]
    fits = {col: _fit_line([r["W"] for r in rows], [r[col] for r in rows]) for col in ("ms_fwd_default", "ms_fwd_tile_skip")}
    return {"L": 8192, "points": rows, "fit_ms_vs_W": fits}


def _fit_line(xs, ys):
    n = len(xs)
    mx, my = sum(xs) / n, sum(ys) / n
    sxx = sum((x - mx) ** 2 for x in xs)
    b = sum((x - mx) * (y - my) for x, y in zip(xs, ys)) / sxx
    a = my - b * mx
    ss_res = sum((y - (a + b * x)) ** 2 for x, y in zip(xs, ys))
    ss_tot = sum((y - my) ** 2 for y in ys) or 1.0
    return {"intercept_ms": a, "slope_ms_per_1024": b * 1024, "r2": 1.0 - ss_res / ss_tot}


def run_mask_builder(steps, warmup, device):
    """Keep-mask construction in front of the operator (not part of `value`): flash_sparse_attn.utils.mask.topk_mask
    through the device kernel, next to the reference's tensor program (masked_fill / topk / zeros / scatter,
    flash_sparse_attn/utils/mask.py:100-110) on the same device, for the bias rows of the benchmark shapes."""
    from flash_sparse_attn.utils import mask as M

    res = []
    for name in ("cfg2", "cfg4", "cfg5"):
        c = CONFIGS[name]
        bias = torch.randn(c["B"], c["Hk"], 1, c["Lk"], generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(device)
        lowest = torch.finfo(torch.bfloat16).min

        def program():
            vals, idx = bias.topk(c["W"], dim=-1, largest=True, sorted=False)
            return torch.zeros_like(bias, dtype=torch.bool).scatter_(-1, idx, vals != lowest)

        with torch.no_grad():
            ms_kernel = time_gpu(lambda: M.topk_mask(bias, None, c["W"], lowest), steps, warmup)
            ms_program = time_gpu(program, steps, warmup)
        res.append({"rows": "%s: %d x %d, top-%d" % (name, c["B"] * c["Hk"], c["Lk"], c["W"]),
                    "us_device_kernel": 1e3 * ms_kernel, "us_tensor_program": 1e3 * ms_program})
    return res


def run_kept_list_handoff(steps, warmup, device):
    """cfg2 forward with a keep-mask that comes from the package's mask builder -- which hands the attention kernels the
    kept columns as index lists with prefix counts, so that the compaction pre-pass has nothing to scan -- next to the
    same mask as a plain bool tensor (not part of `value`)."""
    from flash_sparse_attn import flash_sparse_attn_func
    from flash_sparse_attn.utils import mask as M

    c = CONFIGS["cfg2"]
    q, k, v, _, bias = make_case(c, device)
    lowest = torch.finfo(torch.bfloat16).min
    with torch.no_grad():
        m_lists = M.topk_mask(bias, None, c["W"], lowest)
        m_plain = m_lists.clone()
        has_lists = M.kept_keys_of(m_lists) is not None
        ms_lists = time_gpu(lambda: flash_sparse_attn_func(q, k, v, m_lists, bias, c["scale"], c["causal"]), steps, warmup)
        ms_plain = time_gpu(lambda: flash_sparse_attn_func(q, k, v, m_plain, bias, c["scale"], c["causal"]), steps, warmup)
    return {"workload": "cfg2 forward, mask from topk_mask", "lists_handed_over": bool(has_lists),
            "ms_fwd_with_lists": ms_lists, "ms_fwd_bool_mask_only": ms_plain}


def run_mask_bits_handoff(steps, warmup, device):
    """cfg3 (a bias and a mask per query row) with a keep-mask that comes from the package's mask builder -- which also
    hands the per-query attention kernels the mask packed to one bit per key -- next to the same mask as a plain bool
    tensor (not part of `value`)."""
    from flash_sparse_attn import flash_sparse_attn_func
    from flash_sparse_attn.utils import mask as M

    c = CONFIGS["cfg3"]
    q, k, v, _, bias = make_case(c, device)
    lowest = torch.finfo(torch.bfloat16).min
    with torch.no_grad():
        m_bits = M.topk_mask(bias, None, c["W"], lowest)
        m_plain = m_bits.clone()
    has_bits = M.mask_bits_of(m_bits) is not None
    scale = c["scale"] if c["scale"] is not None else c["D"] ** -0.5
    res = {"workload": "cfg3, mask from topk_mask", "bits_handed_over": bool(has_bits)}
    for name, m in (("with_bits", m_bits), ("bool_mask_only", m_plain)):
        with torch.no_grad():
            res["ms_fwd_" + name] = time_gpu(lambda: flash_sparse_attn_func(q, k, v, m, bias, scale, c["causal"]), steps, warmup)
        qg, kg, vg, bg = [t.detach().clone().requires_grad_(True) for t in (q, k, v, bias)]
        dout = torch.ones_like(q)

        def step():
            for t in (qg, kg, vg, bg):
                t.grad = None  # (no accumulation pass over the 1 GiB bias gradient inside the timed region)
            flash_sparse_attn_func(qg, kg, vg, m, bg, scale, c["causal"]).backward(dout)

        res["ms_fwd_bwd_" + name] = time_gpu(step, steps, warmup)
    return res


def run_bias_producer(steps, warmup, device):
    """The bias producer in front of the operator (not part of `value`): flash_sparse_attn.utils.bias.dynamic_mask_bias
    (one kernel forwards, two backwards) next to the tensor program of the reference's Doge caller
    (examples/modeling/modeling_doge.py:217-222: linear, softplus, multiply, transpose, cast) for the value states of cfg2."""
    import torch.nn.functional as F
    from flash_sparse_attn.utils.bias import dynamic_mask_bias

    c = CONFIGS["cfg2"]
    g = torch.Generator().manual_seed(3)
    K = c["Hk"] * c["D"]
    v = torch.randn(c["B"], c["Lk"], c["Hk"], c["D"], generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
    w = (torch.randn(c["Hk"], K, generator=g) / K ** 0.5).to(torch.bfloat16).to(device).requires_grad_(True)
    a = torch.ones(c["Hk"]).to(torch.bfloat16).to(device).requires_grad_(True)
    gout = torch.randn(c["B"], c["Hk"], 1, c["Lk"], generator=g).to(torch.bfloat16).to(device)

    def program(v_, w_, a_):
        dt = F.linear(v_.reshape(c["B"], c["Lk"], -1), w_)
        return (a_ * F.softplus(dt)).transpose(-1, -2).unsqueeze(-2).to(v_.dtype)

    def fwd_bwd(fn):
        def run():
            fn(v, w, a).backward(gout)
            v.grad = w.grad = a.grad = None
        return run

    res = {"shape": "cfg2 value states: %d x %d x %d x %d" % (c["B"], c["Lk"], c["Hk"], c["D"])}
    with torch.no_grad():
        res["us_fwd_kernel"] = 1e3 * time_gpu(lambda: dynamic_mask_bias(v, w, a), steps, warmup)
        res["us_fwd_tensor_program"] = 1e3 * time_gpu(lambda: program(v, w, a), steps, warmup)
    res["us_fwd_bwd_kernels"] = 1e3 * time_gpu(fwd_bwd(dynamic_mask_bias), steps, warmup)
    res["us_fwd_bwd_tensor_program"] = 1e3 * time_gpu(fwd_bwd(program), steps, warmup)
    return res


def run_ragged_batch(steps, warmup, device):
    """flash_sparse_attn_varlen_func (no mask, no bias, causal) on a ragged batch of 16384 tokens, H=32, Hkv=8, d=128;
    FLOPs are the element-exact causal ones, 4 * d * H * sum(n * (n + 1) / 2)."""
    from flash_sparse_attn import flash_sparse_attn_varlen_func

    lens = [100, 3000, 777, 5000, 64, 2048, 1, 5394]
    H, Hk, D = 32, 8, 128
    g = torch.Generator().manual_seed(2)
    total = sum(lens)
    q = torch.randn(total, H, D, generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
    k = torch.randn(total, Hk, D, generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
    v = torch.randn(total, Hk, D, generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=device)
    dout = torch.ones_like(q)
    flops = float(sum(4 * D * H * (n * (n + 1) // 2) for n in lens))
    with torch.no_grad():
        ms_fwd = time_gpu(lambda: flash_sparse_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens), None, True), steps, warmup)

    def step():
        flash_sparse_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens), None, True).backward(dout)
        q.grad = k.grad = v.grad = None

    ms_fb = time_gpu(step, max(2, steps // 2), max(1, warmup // 2))
    return {"seqlens": lens, "heads": H, "kv_heads": Hk, "head_dim": D, "ms_fwd": ms_fwd, "tflops_fwd": flops / ms_fwd / 1e9,
            "ms_fwd_bwd": ms_fb, "tflops_fwd_bwd": 3.5 * flops / ms_fb / 1e9}


def run_sweeps(steps, warmup, device):
    """Runtime against the window W and against the sequence length L (the reference's claim: README.md:181-191,
    benchmarks/forward_performance.py:661-718), for both paths of the column-mask kernels.  Shapes: H=32, Hkv=8, d=128,
    bias [1,8,1,L], mask = top-W of the bias per row, causal.  W sweep at L=8192; L sweep at W=1024.  A least-squares
    line ms = a + b * x is fitted to every column."""
    fit = _fit_line

    def sweep(points, key):
        rows = []
        for c in points:
            CONFIGS["_sweep"] = c
            row = {"L": c["Lq"], "W": c["W"]}
            for compact, tag in ((True, "compacted"), (False, "tile_skip")):
                r = run_config("_sweep", steps, warmup, device, compact)
                row["ms_fwd_" + tag] = r["ms_fwd"]
                row["ms_fwd_bwd_" + tag] = r["ms_fwd_bwd"]
                row["n_exec_" + tag] = r["n_exec"]
            rows.append(row)
        del CONFIGS["_sweep"]
        fits = {col: fit([r[key] for r in rows], [r[col] for r in rows])
                for col in ("ms_fwd_compacted", "ms_fwd_bwd_compacted", "ms_fwd_tile_skip", "ms_fwd_bwd_tile_skip")}
        return {"points": rows, "fit_ms_vs_" + key: fits}

    def cfg(L, W):
        return dict(B=1, Lq=L, Lk=L, H=32, Hk=8, D=128, bias=(1, 8, 1, L), W=W, causal=True, bwd=True, scale=None)

    return {"w_sweep": sweep([cfg(8192, W) for W in (256, 512, 1024, 2048, 4096, 8192)], "W"),
            "l_sweep": sweep([cfg(L, 1024) for L in (2048, 4096, 8192, 16384, 32768)], "L")}


def cpu_baseline(device_cfg="cfg2", groups=8, chunk=2):
    """The fp32 safe-eager restatement (oracle/eager.py, a port of the reference's eager formula) timed
    on the host cores for a bounded sample of the headline workload: `groups` KV groups (each with its
    4 query heads) of the 8, full sequence length, `chunk` groups at a time (the eager formula materialises
    the [heads, Lq, Lk] fp32 score tensor: 2 groups are 2 GiB per temporary)."""
    from oracle import eager

    c = dict(CONFIGS[device_cfg])
    q, k, v, mask, bias = make_case(c, "cpu")
    G = c["H"] // c["Hk"]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dt, n_exec = 0.0, 0
    with torch.no_grad():
        for g0 in range(0, groups, chunk):
            g1 = min(groups, g0 + chunk)
            qs, ks, vs = q[:, :, G * g0:G * g1].float(), k[:, :, g0:g1].float(), v[:, :, g0:g1].float()
            ms_, bs = mask[:, g0:g1], bias[:, g0:g1].float()
            t0 = time.perf_counter()
            eager.attention_forward(qs, ks, vs, ms_, bs, c["scale"], c["causal"])
            dt += time.perf_counter() - t0
            n_exec += count_tiles(ms_, c["Lq"], c["Lk"], c["causal"], G * (g1 - g0))[0]
    tfl = 4.0 * 64 * 64 * c["D"] * n_exec / dt / 1e12
    return {"value": tfl, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{groups} of {c['Hk']} KV groups ({G * groups} query heads) of {device_cfg} forward, fp32 eager on host, "
                      f"{dt:.2f} s; FLOPs counted on the executed 64x64 tiles of the original layout, as in tile_skip_path "
                      f"(the host computes dense masked attention)",
            "ms_scaled_to_full": dt * 1e3 * c["Hk"] / groups}


def run_secondary_legs(out, legs, args, device, compact, bwd, half):
    """Every default leg but the headline: the tile-skipping path and the all-zero operands of cfg2, the matrix-pipe
    probe, cfg3 / cfg4 / cfg5 with their roofline blocks and the forward W sweep."""
    if compact and "tile_skip" in legs:
        # the same workload through the tile-skipping kernel alone (one kernel per call, no pre-pass)
        ts = run_config("cfg2", *half, device, compact=False, backward=False)
        out["tile_skip_path"] = {"ms_fwd": ts["ms_fwd"], "n_exec_tiles": ts["n_exec"], "tflops_fwd": ts["tflops_fwd"],
                                 "frac_of_peak": ts["tflops_fwd"] / PEAK_BF16_TFLOPS,
                                 "kernel": "fdma::fwd_colmask_kernel<bf16, 128, causal> (compact_mode = never)"}
    if compact and "zero" in legs:
        # The same launches on all-zero Q / K / V / bias: identical mask, tiles and instruction stream.  The device lowers
        # its clocks under the switching activity of real operands (a register-fed MFMA loop reaches 2.4 PFLOP/s on
        # constant operands and 1.9 on random ones), so this is what the kernels' schedule sustains when it does not.
        tz = run_config("cfg2", *half, device, compact=False, backward=False, zero_inputs=True)
        out.setdefault("tile_skip_path", {})["zero_operands"] = {"ms_fwd": tz["ms_fwd"], "tflops_fwd": tz["tflops_fwd"],
                                                                 "frac_of_peak": tz["tflops_fwd"] / PEAK_BF16_TFLOPS}
        cz = run_config("cfg2", *half, device, compact=True, backward=bwd, zero_inputs=True)
        out["zero_operands"] = {"ms_fwd": cz["ms_fwd"], "tflops_fwd": cz["tflops_fwd"],
                                "frac_of_peak": cz["tflops_fwd"] / PEAK_BF16_TFLOPS, "ms_fwd_bwd": cz.get("ms_fwd_bwd"),
                                "note": "same mask, tiles and instruction stream as the headline figures, all-zero Q / K / V / "
                                        "bias: what the schedule sustains when the device does not lower its clock"}
    if "probe" in legs:
        probe = run_mfma_probe()
        if probe is not None:
            out["mfma_probe"] = probe
        probe = run_hbm_probe()
        if probe is not None:
            out["hbm_probe"] = probe
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    # The other benchmark configurations, each against the roofline that bounds it: cfg3 (a bias and a mask per query
    # row, with its dBias) and cfg5 (decode) against HBM, cfg4 (long sequence, narrow window) against the matrix pipe.
    quarter = (max(3, args.steps // 4), max(1, args.warmup // 2))
    configs = {}
    for name in ("cfg3", "cfg4", "cfg5"):
        if name not in legs:
            continue
        if name == "cfg5":  # (a call of some 20 us: many steps, or the two events' own resolution shows)
            r = run_config(name, 10 * args.steps, 2 * args.warmup, device, compact, backward=False)
            r["ms_fwd_c_abi"] = time_decode_c_abi(name, 10 * args.steps, 2 * args.warmup, device)
        else:
            r = run_config(name, *quarter, device, compact, backward=bwd)
        c2 = CONFIGS[name]
        r["workload"] = "%s: B=%d Lq=%d Lk=%d H=%d Hkv=%d d=%d bias%s top-%d%s" % (
            name, c2["B"], c2["Lq"], c2["Lk"], c2["H"], c2["Hk"], c2["D"], list(c2["bias"]), c2["W"], " ∩ causal" if c2["causal"] else "")
        r["roofline"] = config_roofline(name, r)
        configs[name] = r
        torch.cuda.empty_cache()
    if configs:
        out["configs"] = configs
    if "w_sweep" in legs:
        out["w_sweep_fwd"] = run_w_sweep_fwd(*quarter, device)


DEFAULT_LEGS = ("cfg2", "tile_skip", "zero", "probe", "cfg3", "cfg4", "cfg5", "w_sweep", "cpu")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--all", action="store_true",
                    help="also: cfg1, mask builder, bias producer, hand-overs, ragged batch, forward + backward sweeps over W and L")
    ap.add_argument("--legs", default=None,
                    help="comma-separated subset of the default legs to run (" + ", ".join(DEFAULT_LEGS) + "); a profile of one "
                         "leg then holds one workload per kernel; without cfg2 the headline workload is not launched at all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-probe", action="store_true", help="skip the matrix-pipe probe (MFMA rate on constant / random operands)")
    ap.add_argument("--no-backward", action="store_true", help="forward legs only")
    ap.add_argument("--no-compact", action="store_true",
                    help="switch the column-compaction path off (compact_mode = never): time the tile-skipping kernels")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="HBM bytes per launch of the dominant kernel from rocprofv3 --pmc runs (reported as roofline.traffic)")
    ap.add_argument("--summarise-pmc", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn the counter CSVs of two rocprofv3 --pmc passes into " + os.path.relpath(TRAFFIC_FILE, ROOT))
    args = ap.parse_args()
    if args.summarise_pmc:
        summarise_pmc(*args.summarise_pmc)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path has no multi-GPU part in this build; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        sys.exit(1)
    legs = set(DEFAULT_LEGS if args.legs is None else [x for x in args.legs.split(",") if x])
    unknown = legs - set(DEFAULT_LEGS)
    if unknown:
        print("unknown legs: " + ", ".join(sorted(unknown)), file=sys.stderr)
        sys.exit(2)
    if args.no_cpu:
        legs.discard("cpu")
    if args.no_probe:
        legs.discard("probe")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    compact = not args.no_compact
    bwd = not args.no_backward
    half = (max(3, args.steps // 2), max(1, args.warmup // 2))
    if "cfg2" not in legs:
        # a profile of single legs: nothing of the headline workload is launched, and the line holds those legs only
        out = {"metric": "single legs of bench.py (no headline value: run without --legs for the benchmark line)", "legs": sorted(legs)}
        run_secondary_legs(out, legs, args, device, compact, bwd, half)
        print(json.dumps(out))
        return
    main_res = run_config("cfg2", args.steps, args.warmup, device, compact, backward=bwd)
    c = CONFIGS["cfg2"]
    if main_res["compacted"]:
        kernel = ("fdma::fwd_stream_kernel<bf16, causal> (compacted keys, tile images), with its pre-pass (compact_scan_image_kernel) "
                  "in the same call: the duration is that of the whole forward call")
        flops_model = ("4*64*64*d per executed 64x64 tile on the compacted key axis (kept columns packed to the front per "
                       "(batch, kv head)); a 64-row query block executes ceil(visible kept columns / 64) tiles")
    else:
        kernel = "fdma::fwd_colmask_kernel<bf16, 128, causal> (tile skipping on the original key axis)"
        flops_model = "4*64*64*d per 64x64 tile of the original layout that holds a kept, causally visible element"
    out = {
        "metric": "fwd effective TFLOP/s on executed 64x64 tiles (L=8192, W=2048, d=128, bf16, GQA 4:1, mask+bias+causal)",
        "value": main_res["tflops_fwd"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_fwd"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "cfg2: B=1 Lq=Lk=8192 H=32 Hkv=8 d=128 bias[1,8,1,8192] top-2048 ∩ causal, forward",
                   "mask_form": main_res["mask_form"], "n_exec_tiles": main_res["n_exec"],
                   "column_compaction": main_res["compacted"], "flops_model": flops_model,
                   "n_exec_tiles_original_layout": main_res.get("n_exec_original_layout", main_res["n_exec"]),
                   "tile_occupancy_original_layout": main_res["tile_occupancy"]},
        "tflops_fwd_elementwise": main_res["tflops_fwd_elementwise"],
        "tflops_fwd_original_layout_tiles": main_res.get("tflops_fwd_original_layout_tiles", main_res["tflops_fwd"]),
        "ms_fwd": main_res["ms_fwd"],
        "ms_fwd_bwd": main_res.get("ms_fwd_bwd"),
        "tflops_fwd_bwd": main_res.get("tflops_fwd_bwd"),
        "roofline": {
            "bound": "mfma",
            "achieved": main_res["tflops_fwd"],
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": main_res["tflops_fwd"] / PEAK_BF16_TFLOPS,
            "traffic": read_traffic(bool(main_res["compacted"])),
            "kernel": kernel,
            "flops_per_launch": 4.0 * 64 * 64 * c["D"] * main_res["n_exec"],
            "duration_ms": main_res["ms_fwd"],
        },
    }
    if main_res.get("ms_fwd_bwd"):
        out["roofline"]["fwd_bwd"] = {"flops_per_call": 14.0 * 64 * 64 * c["D"] * main_res["n_exec"], "duration_ms": main_res["ms_fwd_bwd"],
                                      "achieved": main_res["tflops_fwd_bwd"], "frac": main_res["tflops_fwd_bwd"] / PEAK_BF16_TFLOPS}
    run_secondary_legs(out, legs, args, device, compact, bwd, half)
    if args.traffic_bytes is not None:
        out["roofline"]["traffic"] = args.traffic_bytes
    quarter = (max(3, args.steps // 4), max(1, args.warmup // 2))
    if args.all:
        out["cfg1"] = run_config("cfg1", *quarter, device, compact)
        out["mask_builder"] = run_mask_builder(*half, device)
        out["bias_producer"] = run_bias_producer(*half, device)
        out["kept_list_handoff"] = run_kept_list_handoff(args.steps, args.warmup, device)
        out["mask_bits_handoff"] = run_mask_bits_handoff(*half, device)
        out["ragged_batch"] = run_ragged_batch(*quarter, device)
        out.update(run_sweeps(*quarter, device))
    if "cpu" in legs:
        out["cpu_baseline"] = cpu_baseline("cfg2", groups=8)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
