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
