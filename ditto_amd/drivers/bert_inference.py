"""The attention blocks of a BERT encoder through task extraction, scheduler binding, build and the
graph engine (reference: benchmark/chimera/cuda/bert_inference.py:15-129).

The reference builds the whole encoder and hands every non-attention layer to its generic
auto-scheduler; only ``multi_head_attention_mma_layer`` goes to the chimera scheduler
(chimera/task_binding.py).  This driver covers that part: a graph of ``n_layers`` attention layers,
each fed by its own packed ``[batch, seq_len, 3 * hidden]`` projection (a graph input standing for
the output of the dense layer in front of it), scheduled, built and timed the way :59-129 do.
"""
import argparse

import ditto_amd as ditto
from ditto_amd import auto_compute as ac
from ditto_amd import auto_schedule, chimera, runtime


def inference(dtype="float16", test=False, batch=1, seq_len=512, hidden=768, n_layers=12, attn_heads=12,
              trials=1000, hip_graph=True, number=600, log_dir=".", scale=None):
    mma_in_dtype, mma_acc_dtype = dtype, "float32"
    mma_MI = mma_NI = mma_KI = 16
    attention = ac.nn.module.MultiHeadAttentionMMA(attn_heads, hidden, mma_in_dtype, mma_acc_dtype, mma_MI, mma_NI,
                                                   mma_KI, scale=scale)
    graph = runtime.Graph([attention.layer(batch, seq_len) for _ in range(n_layers)],
                          outputs=[(i, 0) for i in range(n_layers)])
    graph = chimera.graph_fusion(graph)

    task_name = f"bert_batch{batch}_seq{seq_len}_hidden{hidden}_heads{attn_heads}_layers{n_layers}_inference_{dtype}_mix_mma"
    schedule_option = auto_schedule.ScheduleOption(
        "hip", trials=trials, task_name=task_name, log_file=f"{log_dir}/{task_name}.log", dtype=dtype,
        mma_in_dtype=mma_in_dtype, mma_acc_dtype=mma_acc_dtype, mma_MI=mma_MI, mma_NI=mma_NI, mma_KI=mma_KI,
        device_name="gpu.hip.MI355X")
    tasks = auto_schedule.extract_tasks_from_graph(graph)
    bound_tasks = chimera.task_binding(tasks)
    if not test:
        schedules = auto_schedule.auto_schedule_bound_tasks(bound_tasks, schedule_option)
    else:
        schedules = auto_schedule.retrieve_schedule_bound_tasks(bound_tasks, schedule_option)

    built_mods = {key: ditto.build(sch, args, "hip") for key, (sch, args) in schedules.items()}
    create = runtime.create_hip_graph_engine if hip_graph else runtime.create_graph_engine
    ge = create(graph, built_mods, "cuda:0")
    ge.compile()
    print("Compile done", flush=True)
    ge.run()
    print("Run done", flush=True)
    outputs = ge.get_outputs()
    cost = ge.timeit(number)
    print("Time cost", cost, "ms")
    return cost, outputs, schedules


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--mode", help="tune or test", choices=["tune", "test"], default="tune")
    parser.add_argument("--dtype", help="precision", choices=["float16", "bfloat16"], default="float16")
    parser.add_argument("--trials", type=int, default=1000)
    parser.add_argument("--batch", type=int, default=1)
    parser.add_argument("--seq_len", type=int, default=512)
    parser.add_argument("--hidden", type=int, default=768)
    parser.add_argument("--n_heads", type=int, default=12)
    parser.add_argument("--n_layers", type=int, default=12)
    parser.add_argument("--eager", action="store_true", help="plain launches instead of a HIP graph replay")
    args = parser.parse_args()
    inference(args.dtype, args.mode == "test", args.batch, args.seq_len, args.hidden, args.n_layers, args.n_heads,
              args.trials, not args.eager)
