"""Host decoder with the `hip` MoE layer swapped in through the operator backend.

The same module tree runs once on the GPU with the ``hip`` backend and once on the CPU with a
backend whose two MoE operators are the oracle's restatement of the reference's PyTorch path; in
fp32 the loss, the logits and the parameter gradients must agree.
"""

import copy

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import hip_backend

pytestmark = pytest.mark.gpu


def _oracle_ops():
    from minitrain_amd.kernels.dense_ops import DenseTorchOps
    from minitrain_amd.model.ops import RouterPostprocessOutput

    class OracleOps(DenseTorchOps):
        name = "oracle"

        def router_postprocess(self, logits, top_k, *, normalize):
            r = O.router_postprocess(logits, top_k, normalize=normalize)
            return RouterPostprocessOutput(r.expert_weights, r.expert_indices, r.probability_per_expert, r.z_loss,
                                           r.entropy)

        def fused_moe(self, x, gate_up_proj, down_proj, top_k_index, top_k_weights):
            return O.fused_moe(x, gate_up_proj, down_proj, top_k_index, top_k_weights)

    return OracleOps()


def _small_cfg():
    from minitrain_amd.model.config import ModelConfig

    return ModelConfig(vocab_size=211, seq_len=48, n_layers=2, n_heads=4, hidden_size=64, intermediate_size=128,
                       tie_word_embeddings=True, num_experts=4, experts_per_token=2)


def _batch(cfg, B=3):
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(0, cfg.vocab_size, (B, cfg.seq_len + 1), generator=g)
    return ids[:, :-1].contiguous(), ids[:, 1:].contiguous()


def test_decoder_fp32_matches_oracle_backend():
    from minitrain_amd.model.decoder import MiniTransformer

    cfg = _small_cfg()
    torch.manual_seed(0)
    cpu_model = MiniTransformer(cfg, _oracle_ops())
    gpu_model = copy.deepcopy(cpu_model)
    gpu_model.ops = hip_backend()
    gpu_model = gpu_model.cuda()
    ids, tgt = _batch(cfg)
    loss_c, logits_c = cpu_model(ids, tgt)
    loss_g, logits_g = gpu_model(ids.cuda(), tgt.cuda())
    assert abs(float(loss_c.detach()) - float(loss_g.detach())) <= 1e-5 * max(1.0, abs(float(loss_c.detach())))
    torch.testing.assert_close(logits_g.cpu(), logits_c, rtol=1e-4, atol=1e-5)
    loss_c.backward()
    loss_g.backward()
    for (name, pc), (_, pg) in zip(cpu_model.named_parameters(), gpu_model.named_parameters()):
        scale = float(pc.grad.abs().max())
        err = float((pg.grad.cpu() - pc.grad).abs().max())
        assert err <= 1e-4 * max(scale, 1e-6), (name, err, scale)
    assert set(gpu_model.last_training_metrics) == set(cpu_model.last_training_metrics)


def test_decoder_bf16_training_steps_reduce_loss():
    from minitrain_amd.model.decoder import MiniTransformer
    from minitrain_amd.train.step import build_optimizer, train_step

    cfg = _small_cfg()
    torch.manual_seed(1)
    model = MiniTransformer(cfg, hip_backend(), activation_dtype=torch.bfloat16).cuda()
    opt = build_optimizer(model, lr=3e-3)
    ids, tgt = _batch(cfg, B=4)
    batch = {"input_ids": ids, "targets": tgt}
    losses = [float(train_step(model, opt, batch)) for _ in range(12)]
    assert all(l == l for l in losses)            # finite
    assert losses[-1] < losses[0] - 0.2, losses   # the same batch is being fitted
    assert all(p.grad is None for p in model.parameters())   # zero_grad(set_to_none=True)
