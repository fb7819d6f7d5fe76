"""Usage example with the same call sequence as upstream's example_usage.py: build inputs,
call attention(), take an MSE loss, backpropagate, print the gradients."""
import torch

from flash_tt_attn import attention

B, H, L, D = 4, 8, 128, 32
dev = "cuda"
q = torch.randn(B, H, L, L, D, dtype=torch.float16, device=dev, requires_grad=True)
k = torch.randn_like(q)   # no requires_grad: their .grad stays None, as upstream
v = torch.randn_like(q)
bias = torch.randn(B, H, L, L, dtype=torch.float16, device=dev, requires_grad=True)

out = attention(q, k, v, bias, 1.0 / (D ** 0.5))
loss = torch.nn.functional.mse_loss(out, torch.randn_like(out))
loss.backward()

for name, t in (("q", q), ("k", k), ("v", v), ("bias", bias)):
    print(name, None if t.grad is None else (tuple(t.grad.shape), float(t.grad.float().abs().mean())))
