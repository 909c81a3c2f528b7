"""GPU: the whole layer path (state reset, selection, sharing, block-sparse attention, pivot update, over two layers)
records into one HIP graph -- nothing in it synchronises with the host, allocates outside torch's capture pool or
depends on host-side values -- and every replay on new inputs gives the bits of the eager run, with eager work and
synchronisations between the replays."""

import types

import pytest
import torch

from shareprefill_amd import synthetic

pytestmark = pytest.mark.gpu


class _Module:
    def __init__(self, cfg, sharing, layer_idx, head_dim):
        self.config, self.attention_sharing, self.layer_idx = cfg, sharing, layer_idx
        self.scaling = head_dim ** -0.5
        self.training, self.attention_dropout = False, 0.0


@pytest.mark.parametrize("block_size,n", [(128, 4096), (32, 1536)])  # (the second: the path of the smaller block sizes)
def test_two_layers_replay_from_a_graph(gpu_device, tmp_path, block_size, n):
    from shareprefill_amd import AttentionSharing, shareprefill_attention_forward

    hq, hkv = 8, 2
    table = synthetic.random_cluster_table(hq, 2, 2, 3)
    path = synthetic.write_cluster_table(table, str(tmp_path / "table.json"))
    # fallback_threshold lifted: layer 1 shares the patterns layer 0's pivots left in the state
    cfg = types.SimpleNamespace(block_size=block_size, min_budget=8 * block_size, max_budget=None, pattern_threshold=0.95,
                                similarity_threshold=0.5, fallback_threshold=1e9, queryaware_threshold=0.1,
                                dense_short_prompts=False)
    sharing = AttentionSharing(path)

    def two_layers(q, k, v):
        sharing.reset_state()
        res = []
        for layer in range(2):
            res.extend(shareprefill_attention_forward(_Module(cfg, sharing, layer, 128), q, k, v, None,
                                                      scaling=128 ** -0.5))
        return res

    inputs = [tuple(t.to(gpu_device) for t in synthetic.planted_qkv(hq, hkv, n, 128, 50 + i, q_head_gain=1.0))
              for i in range(3)]
    eager = [[t.clone() for t in two_layers(*x)] for x in inputs]
    hist = sharing.decision_histogram()
    assert hist["dense_pivot"] == 2 and hist["shared"] >= 1
    assert not torch.equal(eager[0][0], eager[1][0])

    sq, sk, sv = (torch.empty_like(t) for t in inputs[0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = two_layers(sq, sk, sv)
    for rep in range(2):
        for i, x in enumerate(inputs):
            for dst, src in zip((sq, sk, sv), x):
                dst.copy_(src)
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip(static_out, eager[i]):
                assert torch.equal(got, want), f"replay {rep}.{i} differs from the eager run"
            two_layers(*inputs[(i + 1) % 3])  # eager work between the replays, on the same state object
