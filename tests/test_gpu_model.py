"""End-to-end generation on a small Llama-3-8B-shaped decoder whose linear, embedding and head weights are
rANS-compressed: the checks the reference makes on whole models -- greedy generation through the runtime
modules (tests/test_rans_pytorch_runtime.py:93-100) and logits against the model on decompressed weights
(tests/test_full_model_rans.py:227-237) -- at two layers, full widths (hidden 4096, FFN 14336, 8 KV
heads, vocabulary 128256), random-init weights from seed 5."""
import pytest
import torch

pytestmark = pytest.mark.gpu

ATOL = RTOL = 1e-2  # the reference's bar against torch.matmul (tests/test_mat_mul.py:220,238)


@pytest.fixture(scope="module")
def small_decoder():
    import bench_model as bm

    dev = torch.device("cuda", 0)
    comp, ref, same, _ = bm.build(2, dev, 1024, 32, "cpu")
    prompt = torch.randint(0, bm.Shape.vocab, (8,), generator=torch.Generator("cpu").manual_seed(6)).to(dev)
    return bm, dev, comp, ref, same, prompt


def test_greedy_ids_equal_the_run_on_decompressed_weights(small_decoder):
    """Sixteen greedy tokens after an eight-token prompt: the compressed model, eager and as one graph replay
    per token, generates the ids of the same decoder on the decompressed bf16 weights contracted in the
    fused kernels' order (the run that differs from it only if a weight bit does)."""
    bm, dev, comp, ref, same, prompt = small_decoder
    n_new, max_len = 16, 8 + 16 + 1
    with torch.no_grad():
        ids_c, _ = bm.generate(bm.Decoder(comp, 2, max_len, dev), prompt, n_new, False)
        ids_g, _ = bm.generate(bm.Decoder(comp, 2, max_len, dev), prompt, n_new, True)
        ids_s, _ = bm.generate(bm.Decoder(same, 2, max_len, dev), prompt, n_new, False)
    assert ids_c == ids_s
    assert ids_g == ids_c
    assert len(set(ids_c)) > 1  # not a degenerate run


def test_logits_match_torch_matmul_on_decompressed_weights(small_decoder):
    """Teacher-forced logits of every step: bit-identical to the same-order run on the decompressed weights
    (what losslessness means for the model), and close to the decoder that runs torch.matmul on them.  The
    two bf16 pipelines add in different orders, and a one-step difference in a bf16 hidden state is carried
    through the layers behind it, so element-wise operator tolerances do not apply to logits; the bar is
    1e-2 relative on the whole logit matrix (Frobenius norm) and four bf16 steps at the largest logit's
    magnitude on every single logit."""
    bm, dev, comp, ref, same, prompt = small_decoder
    n_new, max_len = 16, 8 + 16 + 1
    with torch.no_grad():
        ids, _ = bm.generate(bm.Decoder(ref, 2, max_len, dev), prompt, n_new, False)
        lr = bm.teacher_forced(bm.Decoder(ref, 2, max_len, dev), prompt, ids)
        lc = bm.teacher_forced(bm.Decoder(comp, 2, max_len, dev), prompt, ids)
        ls = bm.teacher_forced(bm.Decoder(same, 2, max_len, dev), prompt, ids)
    assert lc.shape == (n_new, bm.Shape.vocab)
    assert torch.equal(lc, ls)
    diff = (lc.float() - lr.float()).abs()
    assert float(diff.norm() / lr.float().norm()) <= RTOL
    ulp = 2.0 ** (torch.floor(torch.log2(lr.float().abs().max())) - 7)
    assert float(diff.max()) <= 4 * float(ulp), (float(diff.max()), float(ulp))
