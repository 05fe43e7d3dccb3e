"""`colossalai_amd` CLI (reference: colossalai/cli — `colossalai run` / `check`).

`colossalai_amd run --nproc_per_node 8 train.py ...` wraps
torch.distributed.run on this node; `--hostfile` fans the same command out
over SSH for multi-node (one torchrun per host, rendezvous on MASTER_ADDR).
"""

import os
import socket
import subprocess
import sys

import click


@click.group()
def cli():
    pass


@cli.command(context_settings=dict(ignore_unknown_options=True))
@click.option("--nproc_per_node", "--nproc-per-node", type=int, default=1)
@click.option("--nnodes", type=int, default=1)
@click.option("--node_rank", type=int, default=0)
@click.option("--master_addr", type=str, default="127.0.0.1")
@click.option("--master_port", type=int, default=29500)
@click.option("--hostfile", type=str, default=None, help="one hostname per line; SSH fan-out")
@click.option("--ssh-port", type=int, default=22)
@click.argument("script", nargs=1)
@click.argument("script_args", nargs=-1, type=click.UNPROCESSED)
def run(nproc_per_node, nnodes, node_rank, master_addr, master_port, hostfile, ssh_port, script, script_args):
    """Launch a distributed training script (one process per GPU over RCCL)."""
    if hostfile:
        with open(hostfile) as f:
            hosts = [h.strip() for h in f if h.strip() and not h.startswith("#")]
        master_addr = hosts[0] if master_addr == "127.0.0.1" else master_addr
        procs = []
        for rank, host in enumerate(hosts):
            cmd = (
                f"cd {os.getcwd()} && {sys.executable} -m torch.distributed.run "
                f"--nnodes {len(hosts)} --node_rank {rank} --nproc-per-node {nproc_per_node} "
                f"--master-addr {master_addr} --master-port {master_port} {script} {' '.join(script_args)}"
            )
            if host in ("localhost", "127.0.0.1", socket.gethostname()):
                procs.append(subprocess.Popen(cmd, shell=True))
            else:
                procs.append(subprocess.Popen(["ssh", "-p", str(ssh_port), host, cmd]))
        rc = 0
        for p in procs:
            rc |= p.wait()
        sys.exit(rc)

    cmd = [
        sys.executable, "-m", "torch.distributed.run",
        "--nnodes", str(nnodes),
        "--node_rank", str(node_rank),
        "--nproc-per-node", str(nproc_per_node),
        "--master-addr", master_addr,
        "--master-port", str(master_port),
        script, *script_args,
    ]
    os.execv(sys.executable, cmd)


@cli.command()
@click.option("-i", "--installation", is_flag=True, default=True)
def check(installation):
    """Environment sanity check (ROCm, RCCL, kernels)."""
    import torch

    print(f"torch: {torch.__version__}")
    print(f"hip: {torch.version.hip}")
    print(f"gpus visible: {torch.cuda.device_count() if torch.cuda.is_available() else 0}")
    try:
        from colossalai_amd import _C  # noqa: F401

        print("colossalai_amd._C (gfx950 HIP kernels): OK")
    except ImportError as e:
        print(f"colossalai_amd._C: MISSING ({e}) — run `python setup.py build_ext --inplace`")
    import colossalai_amd

    print(f"colossalai_amd: {colossalai_amd.__version__}")


@cli.command()
@click.option("--model", "model_dir", required=True, help="folder with config.json and model.safetensors")
@click.option("--prompt-ids", required=True, help="comma-separated token ids; ';' between prompts")
@click.option("--max-new-tokens", type=int, default=32)
@click.option("--dtype", type=click.Choice(["bfloat16", "float32"]), default="bfloat16")
@click.option("--temperature", type=float, default=0.0, help="0 = greedy")
@click.option("--top-k", type=int, default=0)
@click.option("--top-p", type=float, default=1.0)
@click.option("--max-batch-size", type=int, default=8)
@click.option("--max-step-tokens", type=int, default=2048, help="token budget of one engine step (chunked prefill)")
def generate(model_dir, prompt_ids, max_new_tokens, dtype, temperature, top_k, top_p, max_batch_size, max_step_tokens):
    """Generate from token ids with any registered model (class chosen by config.json)."""
    import json

    import torch

    from colossalai_amd.inference import ContinuousBatchEngine, GenerationConfig, InferenceConfig
    from colossalai_amd.models import load_pretrained

    td = torch.float32 if dtype == "float32" else torch.bfloat16
    device = "cuda" if torch.cuda.is_available() else "cpu"
    model = load_pretrained(model_dir, dtype=td, device=device)
    prompts = [[int(t) for t in part.split(",") if t.strip()] for part in prompt_ids.split(";") if part.strip()]
    longest = max(len(p) for p in prompts)
    engine = ContinuousBatchEngine(
        model, InferenceConfig(max_batch_size=max_batch_size, max_input_len=longest, max_output_len=max_new_tokens, dtype=td),
        max_step_tokens=max_step_tokens)
    gen = GenerationConfig(max_new_tokens=max_new_tokens, do_sample=temperature > 0, temperature=max(temperature, 1e-5),
                           top_k=top_k, top_p=top_p)
    for p, out in zip(prompts, engine.generate(prompts, gen)):
        print(json.dumps({"prompt_ids": p, "output_ids": out[len(p):]}))


@cli.command(context_settings=dict(ignore_unknown_options=True))
@click.argument("args", nargs=-1, type=click.UNPROCESSED)
def replay(args):
    """Replay a token trace through the serving engine and write logits (see `replay --help-trace`;
    arguments as bin/trace_run: --model DIR --dtype T --out DIR --max-tokens N, steps on stdin)."""
    from colossalai_amd.inference.trace_replay import main as replay_main

    sys.exit(replay_main(["--help"] if "--help-trace" in args else list(args)))


@cli.command()
def models():
    """List the architectures the model registry can load."""
    from colossalai_amd.models import registered_models

    print("\n".join(registered_models()))


if __name__ == "__main__":
    cli()
