"""The MLP demo (the reference's tests/python/test_model_demo.py on synthetic samples): it must learn
its task on every layer kind, and inference from the exported bit-packed weight files must give the
same predictions as inference from the float weights."""
import pytest
import torch

import mlp_demo


def test_dataset_shape_and_labels():
    ds = mlp_demo.synthetic_dataset(100, seed=3)
    x, y = ds.tensors
    assert tuple(x.shape) == (96, 512) and x.dtype == torch.float16          # whole batches of 32
    assert set(x.unique().tolist()) == {-0.5, 0.5} and set(y.unique().tolist()) <= {0.0, 1.0}
    assert torch.equal(y.bool(), x[:, :64].float().sum(1) > x[:, 64:128].float().sum(1))
    assert 0.3 < float(y.float().mean()) < 0.7


@pytest.mark.parametrize("model", ["bnn_fp16", "nn_elastic"])
def test_torch_path_models_learn_on_cpu(model):
    r = mlp_demo.run(model, epochs=3, train_samples=8192, test_samples=1024, device="cpu", log=lambda s: None)
    assert r["history"][-1][0] < r["history"][0][0] and r["accuracy"] > 0.85


def test_bgemm_models_refuse_cpu():
    with pytest.raises(RuntimeError):
        mlp_demo.run("bgemm", epochs=0, device="cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["bgemm_elastic", "bgemm_bireal", "bgemm"])
def test_bgemm_models_learn_and_run_from_packed_files(model, tmp_path):
    r = mlp_demo.run(model, epochs=4, train_samples=16384, test_samples=2048, device="cuda:0",
                     export=str(tmp_path), log=lambda s: None)
    assert r["history"][-1][0] < r["history"][0][0] and r["accuracy"] > 0.85
    if model == "bgemm_elastic":
        assert r["packed_files"] == {}                 # ternary activations, learned scales: nothing sign-packed to export
        return
    assert sorted(r["packed_files"]) == ["lin2", "lin3"]
    assert r["accuracy_from_packed"] == r["accuracy"]
    # same logits, bit for bit, with the float weights gone
    mlp, (x, _) = r["mlp"], next(iter(r["test_loader"]))
    x = x.to("cuda:0").float()
    with torch.no_grad():
        want = mlp(x)
        for lin in (mlp.lin2, mlp.lin3):
            lin.weight.data = torch.full_like(lin.weight, float("nan"))
            lin.use_packed_weight(lin._wp)
        assert torch.equal(mlp(x), want)


@pytest.mark.gpu
def test_kernel_and_torch_elastic_layers_train_alike():
    a = mlp_demo.run("bgemm_elastic", epochs=2, train_samples=4096, test_samples=512, device="cuda:0", log=lambda s: None)
    b = mlp_demo.run("nn_elastic", epochs=2, train_samples=4096, test_samples=512, device="cuda:0", log=lambda s: None)
    assert abs(a["history"][-1][0] - b["history"][-1][0]) < 0.05 and abs(a["accuracy"] - b["accuracy"]) < 0.05


@pytest.mark.gpu
def test_binary_self_attention_block_kernels_equal_dense_torch():
    """The BERT self-attention block with both matmuls on the binary kernels gives, bit for bit, what dense torch
    matmuls on the de-binarised tensors give; gradients reach every projection."""
    import attention_demo
    torch.manual_seed(12)
    block = attention_demo.BinarySelfAttention(hidden_size=768, num_attention_heads=12).to("cuda:0")
    x = torch.randn(2, 128, 768, device="cuda:0")
    mask = torch.zeros(2, 1, 1, 128, device="cuda:0")
    mask[1, :, :, 100:] = -10000.0                       # padded tail of the second sequence
    with torch.no_grad():
        block(x, mask)                                   # initialises the layers' scales
        out_k, scores_k = block(x, mask)
        block.kernels = False
        out_t, scores_t = block(x, mask)
        block.kernels = True
    assert tuple(out_k.shape) == (2, 128, 768) and tuple(scores_k.shape) == (2, 12, 128, 128)
    assert torch.equal(scores_k, scores_t) and torch.equal(out_k, out_t)
    assert int((scores_k[0] * 8).round().abs().max()) <= 64      # scores are integers in [-64, 64] over sqrt(64)
    out, _ = block(x, mask)
    # a loss with gradients of order one: the Functions' backward runs in fp16, as the reference's does
    (out.float() * torch.randn_like(out)).sum().backward()
    for lin in (block.query, block.key, block.value, block.dense):
        assert lin.weight.grad is not None and torch.isfinite(lin.weight.grad).all() and lin.weight.grad.abs().sum() > 0
