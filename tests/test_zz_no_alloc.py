"""The allocation-free entry point af3_batch_diffusion_self_attention_forward_static
(scratch in a device array the library owns) against the workspace-taking entry
point it is a variant of: same kernels, so the outputs must be bit-identical.

Two calls in a row, the second on a smaller problem (the array then still holds
the larger call's data beyond what the second call writes), then a call beyond
the array's size, which must be refused without enqueuing anything.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(pkg, seed, batch, seq, channels, heads, masked, out_dtype):
    d = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, seq, channels, generator=g).bfloat16().to(d)
    w = (torch.randn(4 * channels, channels, generator=g) * 0.05).bfloat16().to(d)
    qb = (torch.randn(channels, generator=g) * 0.1).to(d)
    mask = (torch.arange(seq) < seq - masked).float().to(d)
    bias = torch.randn(heads, seq, seq, generator=g).to(d)
    want = pkg.ops.batch_diffusion_self_attention(x, mask, bias, w, qb, heads, out_dtype=out_dtype)
    out = torch.full_like(want, float("nan"))
    before = torch.cuda.memory_allocated(d)
    got = pkg.ops.batch_diffusion_self_attention(x, mask, bias, w, qb, heads, out_dtype=out_dtype, out=out,
                                                 static_scratch=True)
    assert torch.cuda.memory_allocated(d) == before        # torch's allocator was not touched either
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr()
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, want), f"static-scratch output differs (batch={batch} seq={seq} c={channels})"


def test_static_scratch_matches_workspace_entry_point_twice(gpu_pkg):
    print("test_static_scratch: 5 x 768 x 768, 16 heads, then 2 x 130 x 384", flush=True)
    _case(gpu_pkg, 1, 5, 768, 768, 16, 60, torch.bfloat16)     # the diffusion transformer's shape: 23.6 MB of scratch
    _case(gpu_pkg, 2, 2, 130, 384, 16, 7, torch.float32)       # smaller, ragged, right after it
    _case(gpu_pkg, 3, 1, 1536, 384, 16, 0, torch.bfloat16)     # the trunk's single attention at 1536 tokens


def test_static_scratch_refuses_what_does_not_fit(gpu_pkg):
    pkg = gpu_pkg
    d = torch.device("cuda:0")
    batch, seq, c, h = 6, 768, 768, 16                         # 28.3 MB would fit; 6 x 1024 x 768 x 8 = 37.7 MB does not
    seq = 1024
    assert batch * seq * c * 8 > pkg.lib.STATIC_SCRATCH_BYTES
    x = torch.zeros(batch, seq, c, dtype=torch.bfloat16, device=d)
    w = torch.zeros(4 * c, c, dtype=torch.bfloat16, device=d)
    out = torch.full((batch, seq, h, c // h), 7.0, dtype=torch.bfloat16, device=d)
    with pytest.raises(pkg.lib.Af3Error, match="exceeds the library-owned scratch"):
        pkg.ops.batch_diffusion_self_attention(x, None, None, w, None, h, out=out, static_scratch=True)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())                            # nothing was enqueued
