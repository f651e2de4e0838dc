"""The command-line driver of the end-to-end sparse attention model: the reference's options
(end2end/sspmm_e2e/end_to_end.py:20-35) are accepted, and on a GPU it prints the reference's result lines."""
import re

import pytest
import torch

from sspmm_amd import end_to_end


def test_options_of_the_reference_script_are_accepted():
    a = end_to_end._parser().parse_args(["--vocab_size", "300", "--num_class", "2", "--mlp_dim", "512", "--embed_dim", "128",
                                         "--num_heads", "2", "--bs", "8", "--seq_len", "1024", "--sparsity", "0.95",
                                         "--vec_length", "8", "--model", "both", "--mem"])
    assert (a.vocab_size, a.mlp_dim, a.embed_dim, a.num_heads, a.bs, a.seq_len, a.sparsity, a.model, a.mem) == \
        (300, 512, 128, 2, 8, 1024, 0.95, "both", True)
    d = end_to_end._parser().parse_args([])  # the reference's defaults
    assert (d.vocab_size, d.mlp_dim, d.embed_dim, d.num_heads, d.bs, d.seq_len, d.sparsity, d.vec_length, d.model) == \
        (257, 1024, 256, 4, 2, 4096, 0.9, 8, "sparse")


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the message on a machine without a GPU")
def test_without_a_gpu_it_says_so():
    with pytest.raises(SystemExit, match="needs a GPU"):
        end_to_end.main([])


@pytest.mark.gpu
def test_prints_a_time_for_each_model(built_library, capsys):
    assert end_to_end.main(["--seq_len", "512", "--embed_dim", "128", "--num_heads", "2", "--mlp_dim", "256", "--bs", "2",
                            "--model", "both", "--graph"]) == 0
    out = capsys.readouterr().out
    assert len(re.findall(r"vectorSparse average runtime [0-9.]+ milliseconds", out)) == 2
    assert len(re.findall(r"dense average runtime [0-9.]+ milliseconds", out)) == 2
    assert end_to_end.main(["--seq_len", "512", "--embed_dim", "128", "--num_heads", "2", "--mlp_dim", "256", "--mem"]) == 0
    assert re.search(r"vectorSparse peak memory [0-9.]+ MB", capsys.readouterr().out)
    with pytest.raises(SystemExit):
        end_to_end.main(["--embed_dim", "100", "--num_heads", "3"])
