"""The step before the hot path on the GPU: a synthetic batch packed by art_amd.pack, written to
and read back from the raw `{key}.pt` files, staged row by row through RowStager (pinned
double buffer, copy stream) and fed to the fused loss.  The loss, the logprobs and d_hidden of
every row must equal, bit for bit, what the same rows give when handed to the GPU directly."""
import random

import pytest
import torch

from art_amd import pack
from art_amd.train import fused_grpo_loss

pytestmark = pytest.mark.gpu


def synthetic_results(n_prompts, n_comp, prompt_len, comp_len, vocab, seed):
    g = random.Random(seed)
    results = []
    for pid in range(n_prompts):
        prompt = [g.randrange(vocab) for _ in range(prompt_len)]
        for _ in range(n_comp):
            n = g.randint(comp_len // 2, comp_len)
            comp = [g.randrange(vocab) for _ in range(n)]
            results.append(pack.TokenizedResult(
                token_ids=prompt + comp, input_pos=list(range(prompt_len + n)),
                assistant_mask=[0] * prompt_len + [1] * n,
                logprobs=[float("nan")] * prompt_len + [-2.0 * g.random() for _ in range(n)],
                advantage=g.uniform(-1, 1), prompt_id=pid, prompt_length=prompt_len))
    return results


def test_pack_roundtrip_stager_fused_loss(artk_lib, gpu, tmp_path):
    print("pack -> dir -> RowStager -> fused loss", flush=True)
    S, H, V = 1024, 128, 4096
    packed = pack.packed_tensors_from_tokenized_results(
        synthetic_results(6, 4, 40, 150, V, 3), S, pad_token_id=V - 1, rng=random.Random(5))
    n_rows = packed["tokens"].shape[0]
    assert n_rows >= 3
    disk = pack.packed_tensors_to_dir(packed, str(tmp_path / "tensors"))
    loaded = pack.packed_tensors_from_dir(**disk)
    for key, t in packed.items():
        a, b = (t, loaded[key]) if not t.is_floating_point() else (t.nan_to_num(7.0), loaded[key].nan_to_num(7.0))
        assert torch.equal(a, b), key

    g = torch.Generator().manual_seed(11)
    hidden = [torch.randn(1, S, H, generator=g).to(torch.bfloat16).to(gpu) for _ in range(n_rows)]
    lm_head = (0.05 * torch.randn(V, H, generator=g)).to(torch.bfloat16).to(gpu)

    def run(row, h):
        hs = h.clone().requires_grad_(True)
        loss, metrics, lp = fused_grpo_loss(hs, lm_head, row["tokens"], row["logprobs"], row["advantages"],
                                            row["assistant_mask"], row["weights"])
        loss.backward()
        return loss.detach().clone(), lp.clone(), hs.grad.clone(), metrics["mask_count"].clone()

    direct = [run({k: v[i:i + 1].to(gpu) for k, v in packed.items()}, hidden[i]) for i in range(n_rows)]
    stager = pack.RowStager(S, gpu)
    staged = []
    for i, row in enumerate(stager.rows(loaded)):
        assert all(t.is_cuda and tuple(t.shape) == (1, S) for t in row.values())
        staged.append(run(row, hidden[i]))
    torch.cuda.synchronize()
    assert len(staged) == n_rows
    for i, (a, b) in enumerate(zip(direct, staged)):
        assert float(a[3]) > 0, "every packed row carries assistant tokens"
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[2], b[2]), i
    # the one-row entry point gives the same tensors
    one = stager.to_device(loaded, n_rows - 1)
    for key, t in packed.items():
        want = t[n_rows - 1:n_rows]
        got = one[key].cpu()
        assert torch.equal(want.nan_to_num(7.0) if want.is_floating_point() else want,
                           got.nan_to_num(7.0) if got.is_floating_point() else got), key
    # a second pass over the same stager (slots are reused) still delivers every row intact
    for i, row in enumerate(stager.rows(loaded)):
        assert torch.equal(row["tokens"].cpu(), packed["tokens"][i:i + 1])
        assert torch.equal(row["assistant_mask"].cpu(), packed["assistant_mask"][i:i + 1])
    # a pass that is abandoned after its first row releases the slot it held: the next pass is intact
    it = stager.rows(loaded)
    first = next(it)
    assert torch.equal(first["tokens"].cpu(), packed["tokens"][0:1])
    it.close()
    for i, row in enumerate(stager.rows(loaded)):
        assert torch.equal(row["tokens"].cpu(), packed["tokens"][i:i + 1])
        assert torch.equal(row["advantages"].cpu(), packed["advantages"][i:i + 1])
