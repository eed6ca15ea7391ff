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


def test_counter_means_per_kernel(tmp_path):
    """A --pmc run's file: a row per dispatch and counter; the table has a kernel's dispatches, their
    mean time and the mean of each counter."""
    os.makedirs(tmp_path / "vm")
    head = ('"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size","Kernel_Id","Kernel_Name",'
            '"Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count","Accum_VGPR_Count","SGPR_Count","Counter_Name","Counter_Value",'
            '"Start_Timestamp","End_Timestamp"\n')
    rows = []
    for d, (name, grid, t0, t1, mfma, cyc) in enumerate([("k_attn_cta(AttnArgs)", 262144, 0, 60000, 100.0, 1000.0),
                                                         ("k_attn_cta(AttnArgs)", 262144, 70000, 110000, 300.0, 3000.0),
                                                         ("k_attn_cta(AttnArgs)", 512, 120000, 121000, 1.0, 10.0),
                                                         ("void k_rmsnorm_v4<unsigned short, unsigned short, 4>(float*)", 524288, 130000, 140000, 0.0, 500.0)]):
        for cname, val in (("SQ_INSTS_MFMA", mfma), ("SQ_CYCLES", cyc)):
            rows.append(f'{d},{d},"Agent 1",1,9,9,{grid},3,"{name}",512,0,0,8,0,32,"{cname}",{val},{t0},{t1}\n')
    (tmp_path / "vm" / "9_counter_collection.csv").write_text(head + "".join(rows))
    got = ps.read_counters(str(tmp_path), min_grid=1024)
    assert got["k_attn_cta"]["us"] == [60.0, 40.0] and got["k_attn_cta"]["SQ_INSTS_MFMA"] == [100.0, 300.0]
    table = ps.counter_table(got, ["k_attn"])
    assert "| `k_attn_cta` | 2 | 50.0 | 2,000 | 200 |" in table and "rmsnorm" not in table
    assert "k_rmsnorm_v4<unsigned short,unsigned short,4>" in ps.counter_table(got, [])
    assert ps.main([str(tmp_path), "--counters", "--kernel", "k_attn", "--grid", "1024"]) == 0
