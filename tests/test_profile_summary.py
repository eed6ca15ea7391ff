"""The per-kernel summary of a profiler trace: which dispatches make a step, and their sums."""
import os

from xyntetik_runner_amd import profile_summary as ps

HEADER = "Kind,Agent_Id,Queue_Id,Kernel_Id,Kernel_Name,Correlation_Id,Start_Timestamp,End_Timestamp,Grid_Size_X\n"


def write_trace(folder, rows):
    os.makedirs(os.path.join(folder, "host"), exist_ok=True)
    with open(os.path.join(folder, "host", "1_kernel_trace.csv"), "w") as f:
        f.write(HEADER)
        for i, (s, e, name, grid) in enumerate(rows):
            f.write(f'KERNEL_DISPATCH,1,1,{i},"{name}",{i},{s},{e},{grid}\n')


def test_the_last_decode_step_and_a_prompt_step(tmp_path):
    rows = [
        (0, 1000, "void k_embedding<__hip_bfloat16>(int*)", 2048 * 256),
        (1000, 31000, "void k_gemm_tile_async<256, 256, 4, 2, 2, true>(GemmArgs)", 65536),
        (31000, 32000, "k_sample(SampleArgs)", 64),
        (40000, 40500, "void k_embedding<__hip_bfloat16>(int*)", 8 * 256),
        (40500, 42500, "void k_gemm_skinny<1, 1, 8, 8, true, true>(GemmArgs)", 16384),
        (42500, 44000, "void k_gemm_skinny<1, 1, 8, 8, true, true>(GemmArgs)", 16384),
        (44000, 44500, "k_sample(SampleArgs)", 64),
        (50000, 50500, "void k_embedding<__hip_bfloat16>(int*)", 8 * 256),
        (50500, 53500, "void k_gemm_skinny<1, 1, 8, 8, true, true>(GemmArgs)", 16384),
        (53500, 54000, "k_sample(SampleArgs)", 64),
    ]
    write_trace(str(tmp_path), rows)
    got = ps.read_trace(str(tmp_path))
    assert len(got) == len(rows) and got[0][2].startswith("void k_embedding")
    assert ps.short_name(rows[1][2]) == "k_gemm_tile_async<256,256,4,2,2,true>"
    # decode steps: from one pick to the next
    steps = ps.spans(got, "k_sample", 0)
    assert steps == [(2, 6), (6, 9)]
    table = ps.summarize(got, *steps[-1])
    assert "3 kernels, span 10 us, kernels busy 4 us" in table
    assert "| 3.0 | 75.0% | 1 x 3.0 | `k_gemm_skinny<1,1,8,8,true,true>` |" in table
    # the prompt step: the embedding of 2,048 rows up to the next embedding
    assert ps.spans(got, "k_embedding", 2048 * 256) == [(0, 3)]
    assert "k_gemm_tile_async<256,256,4,2,2,true>" in ps.summarize(got, 0, 3)
