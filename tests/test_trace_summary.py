"""The per-kernel summary of a profiler database: steps are cut between embedding kernels."""
import sqlite3

from holon_amd import trace_summary


def _database(path, names):
    db = sqlite3.connect(path)
    db.execute("create table rocpd_info_kernel_symbol (id integer, kernel_name text)")
    db.execute("create table rocpd_kernel_dispatch (kernel_id integer, start integer, end integer, grid_size_x integer, "
               "grid_size_y integer, grid_size_z integer, workgroup_size_x integer)")
    ids = {}
    t = 1000
    for name, us in names:
        if name not in ids:
            ids[name] = len(ids) + 1
            db.execute("insert into rocpd_info_kernel_symbol values (?, ?)", (ids[name], name))
        db.execute("insert into rocpd_kernel_dispatch values (?, ?, ?, 512, 2, 1, 256)", (ids[name], t, t + us * 1000))
        t += us * 1000 + 500
    db.commit()
    db.close()


def test_steps_are_cut_between_embedding_kernels(tmp_path, capsys):
    step = lambda a, b: [("_Z16embedding_kernelItEvPKi(args)", 5), ("_Z18attn_decode_kernelILi128EEv8AttnArgs.kd", a),
                         ("_Z18attn_decode_kernelILi128EEv8AttnArgs.kd", a), ("_Z13argmax_kernelPKfPii.kd", b)]
    path = str(tmp_path / "t_results.db")
    _database(path, step(100, 7) + step(20, 8) + step(30, 9) + step(40, 10))
    assert trace_summary.main([path, "--step", "decode"]) == 0
    text = capsys.readouterr().out
    assert "one decode step: 4 kernels, 0.053 ms of kernel time" in text          # the third step from the end: 5 + 2 * 20 + 8
    rows = [line.split() for line in text.splitlines()[2:]]
    assert rows[0][:4] == ["40.0", "75.5%", "2", "20.0"] and rows[0][4].startswith("attn_decode<128") and "grid 2x2x1" in text
    assert trace_summary.main([path, "--step", "prefill", "--index", "0"]) == 0
    assert "one prompt step: 4 kernels, 0.212 ms" in capsys.readouterr().out
    assert trace_summary.main([path]) == 0
    assert "whole run: 16 kernels" in capsys.readouterr().out
    assert trace_summary.main([path, "--step", "prefill", "--index", "9"]) == 1


def test_a_step_by_class_of_kernel(tmp_path, capsys):
    """`--classes`: the step's kernel time under attention, matrix products, elementwise, sampling and the rest, each as
    a share of the step from first start to last end; the remainder is the gaps between kernels."""
    step = [("_Z16embedding_kernelItEvPKi(args)", 5), ("_Z18attn_decode_kernelILi128ELb1EEv8AttnArgs.kd", 30),
            ("_Z17attn_merge_kernelILi128EEvPKf.kd", 10), ("_Z18gemm_skinny_kernelILi1ELi16E.kd", 40),
            ("Cijk_Alik_Bljk_BBS_BH_Bias_HA_S_SAV_UserArgs_MT128x256x64", 20), ("_Z18rmsnorm_row_kernelItLb1E.kd", 4),
            ("_Z13argmax_kernelPKfPii.kd", 6), ("__amd_rocclr_copyBuffer.kd", 3)]
    path = str(tmp_path / "c_results.db")
    _database(path, step * 4)
    assert trace_summary.main([path, "--step", "decode", "--classes"]) == 0
    lines = capsys.readouterr().out.splitlines()
    table = {" ".join(line.split()[2:]): float(line.split()[0]) for line in lines[lines.index(next(
        l for l in lines if l.strip().startswith("us"))) + 1:]}
    assert table == {"matrix products": 60.0, "attention": 40.0, "elementwise": 9.0, "sampling": 6.0,
                     "other (copies, library elementwise)": 3.0, "between kernels": 3.5}
    assert trace_summary.kernel_class("_ZN12_GLOBAL__N_116gemm_rows_kernelILi4E") == "matrix products"
