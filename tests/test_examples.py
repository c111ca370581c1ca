"""The restated example scripts: same flags, same final stdout lines as the reference's (its test runner
greps them, examples/bench_test.sh:284-285)."""
import pytest

pytestmark = pytest.mark.gpu


def test_fine_grained_example(capsys):
    from tilelang_ascend_amd.examples.dequantize_gemm import example_dequant_gemm_fine_grained as ex

    ex.main(["--m", "128", "--n", "256", "--k", "512", "--input-dtype", "bfloat16", "--some-unknown-flag", "1"])
    out = capsys.readouterr().out
    assert "Unknown args: ['--some-unknown-flag', '1']" in out
    assert "INT4 -> FP16 unpack test passed!" in out and "INT8 Test passed: M=128, N=256, K=512, output=int32" in out
    assert out.rstrip().splitlines()[-2] == "Kernel Output Match!" and "All tests passed!" in out


def test_w4a8_example(capsys):
    from tilelang_ascend_amd.examples.dequantize_gemm import example_dequant_gemm_w4a8 as ex

    ex.main([])
    out = capsys.readouterr().out
    assert out.count("Test passed:") == 3 and out.rstrip().endswith("Test Passed!")
    ex.main(["--M", "40", "--N", "20", "--K", "64"])
    assert "Test passed: M=40, N=20, K=64" in capsys.readouterr().out


def test_quant_matmul_examples(capsys):
    from tilelang_ascend_amd.examples.quant_batch_matmul import example_quant_batch_matmul as exb
    from tilelang_ascend_amd.examples.quant_batch_matmul import example_quant_matmul as ex2

    exb.main(["--b", "2", "--m", "256", "--n", "512", "--k", "256"])
    out = capsys.readouterr().out
    assert out.rstrip().splitlines()[-2:] == ["QuantBatchMatmul example passed!", "Kernel Output Match!"]
    ex2.main(["--m", "256", "--n", "512", "--k", "256"])
    out = capsys.readouterr().out
    assert out.rstrip().splitlines()[-2:] == ["QuantMatmul example passed!", "Kernel Output Match!"]


def test_deepseek_v4_examples(caplog):
    import logging

    from tilelang_ascend_amd.examples.deepseek_v4 import act_quant, int8_gemm

    with caplog.at_level(logging.INFO):
        act_quant.test()
        int8_gemm.test()
    msgs = [r.getMessage() for r in caplog.records]
    assert msgs.count("init successful!") == 2 and msgs.count("Kernel Output Match!") == 2
