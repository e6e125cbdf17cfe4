"""Replay a trace of token steps through the engine and write the logits it asks for.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line: {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.
For a step that wants logits, OUT/<n>.f32 receives them as little-endian fp32 [wanted, vocab]; after every step the
line `done <n>` is printed.  The model class comes from DIR/config.json like everywhere else in the engine; the KV pool
holds --max-tokens tokens and --max-requests request rows (4), so slots and rows are reused as requests end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens that live requests hold at most, together")
    ap.add_argument("--max-requests", type=int, default=4, help="requests that are live at most")
    ap.add_argument("--disable-cuda-graph", action="store_true", help="run decode steps eagerly")
    args = ap.parse_args(argv)

    import torch
    from semi_pd_amd.entrypoints.engine import _build_runner
    from semi_pd_amd.managers.replay_scheduler import ReplayScheduler
    from semi_pd_amd.semi_pd.utils import InstanceRole
    from semi_pd_amd.server_args import ServerArgs

    if not torch.cuda.is_available():
        print("trace_run needs a HIP device: the engine has no host path", file=sys.stderr)
        return 2
    # fp32 means fp32: no reduced-precision matrix mode
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    os.makedirs(args.out, exist_ok=True)
    n = max(64, int(args.max_tokens))
    sa = ServerArgs(model_path=args.model, load_format="auto", dtype=args.dtype, context_length=n, max_total_tokens=n,
                    max_running_requests=args.max_requests, cuda_graph_max_bs=args.max_requests,
                    disable_cuda_graph=args.disable_cuda_graph, skip_tokenizer_init=True, enable_semi_pd=False)
    mr = _build_runner(sa, sa.base_gpu_id, 0, InstanceRole.OTHER, (sa.nccl_port_base or 29600) + 3,
                       max_total_tokens=sa.max_total_tokens)
    mr.init_attention_backend()
    mr.init_cuda_graphs()
    sched = ReplayScheduler(sa, mr)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = sched.replay_step(step.get("entries", []), step.get("end", []))
        if logits is not None:
            data = logits.to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, f".{step['step']}.f32.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(args.out, f"{step['step']}.f32"))
        else:
            torch.cuda.synchronize()
        print(f"done {step['step']}", flush=True)
    torch.cuda.synchronize()
    return 0


if __name__ == "__main__":
    sys.exit(main())
