"""GPU: one speculation (all draft levels) replayed from a captured graph with the prefix length in device memory,
against the same speculation issued eagerly.  The graph is replayed several times, for growing prefixes, with eager
work (a target forward, verification, compaction) and synchronizations in between, and every replay is compared with
the eager result for its prefix."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from subspec_amd.cache import create_kv_cache
from subspec_amd.draft import SubSpecSDDraftModel
from subspec_amd.generator import SubSpecSDGenerator
from subspec_amd.model import DecoderConfig, build_models, init_weights
from subspec_amd.utils import DraftParams
from subspec_amd.wandb_logger import wandb_logger

DEV = "cuda:0"
CFG = DecoderConfig(num_hidden_layers=4, hidden_size=256, num_attention_heads=2, num_key_value_heads=1,
                    head_dim=128, intermediate_size=512, vocab_size=2048)


def _tree_lists(tree):
    d = tree.get_tree_data()
    return d["token_ids"].tolist(), d["parent_indices"].tolist(), d["cumulative_probabilities"].float().tolist()


def test_replayed_speculation_equals_the_eager_one():
    w = init_weights(CFG, 5, DEV)
    kv = create_kv_cache("static", max_cache_len=1024, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv, device=DEV, weights=w)
    g = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, CFG.vocab_size, (300,), generator=g).to(DEV)
    target.prefill(prompt, 0)
    dm = SubSpecSDDraftModel(draft)
    dm.draft_params = DraftParams(temperature=0.2, max_depth=5, topk_len=4)
    dm.set_past_key_values(kv)
    dm.capture_graphs, dm.graph_warmup = True, 1
    root = torch.tensor([[7]], device=DEV)
    # prefixes inside one bucket (<= 256 and <= 512), visited out of order; the cache holds valid rows up to 300
    from subspec_amd.cpu_tree import Tree
    for step, prefix in enumerate([200, 203, 250, 201, 290, 300, 260]):
        print("draft graph: prefix", prefix, flush=True)
        kv.seq_len = prefix
        dm.capture_graphs = False
        plain = _tree_lists(dm.speculate(root + step))       # launches laid out for the actual prefix length
        # the same launches the graph holds (laid out for the bucket's upper bound, prefix length read on the device),
        # issued eagerly: what a replay must reproduce bit for bit
        dm.prefix_len = prefix
        dm.capture_graphs = True
        bound = dm._graph_bound()
        assert bound == (256 if prefix < 256 else 512)
        dm.tree = Tree(int(root + step), draft.dtype)
        dm._grow_levels((root + step)[0], bound, torch.tensor([prefix], dtype=torch.int64, device=DEV))
        want = _tree_lists(dm.update_tree())
        saved = kv.cache.data.clone()
        # eager work between two replays: a target forward over other rows, a synchronization
        target.prefill(prompt[:5], 600)
        torch.cuda.synchronize()
        got = _tree_lists(dm.speculate(root + step))
        assert dm.graph_replays == step + 1                  # the eager speculations above were the warm-up
        assert got == want, prefix
        assert torch.equal(kv.cache.data[..., :590, :], saved[..., :590, :]), prefix     # and wrote the same draft rows
        # against the plain call only rounding may differ (other key chunks): the first level's candidates agree
        assert got[0][1:5] == plain[0][1:5] and got[2][1:5] == pytest.approx(plain[2][1:5], rel=0.2, abs=2e-3), prefix      # temperature 0.2 turns a bf16 rounding of a logit into a few percent
    assert len(dm._graphs) == 2                              # one graph per bucket: prefixes up to 256, up to 512


def test_cycle_with_graph_replay_emits_the_targets_tokens():
    w = init_weights(CFG, 9, DEV)
    outs = {}
    for graph in (False, True):
        kv = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
        target, draft, _ = build_models(CFG, kv, device=DEV, weights=w, first_streamed=2)
        gen = SubSpecSDGenerator(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=4, topk_len=4),
                                 generator_kwargs=dict(verify_method="exact", draft_graph=graph))
        gen.draft_model.graph_bucket = 32                    # several buckets within one generation
        prompt = torch.randint(0, CFG.vocab_size, (1, 40), generator=torch.Generator().manual_seed(4)).to(DEV)
        wandb_logger.clear_log_data()
        outs[graph] = gen.generate(prompt, max_new_tokens=60, do_sample=False, past_key_values=kv)[0].cpu()
        if graph:
            assert gen.draft_model.graph_replays >= wandb_logger.log_data["n_iter"] - 2 and len(gen.draft_model._graphs) >= 2
        assert kv.get_seq_length() == 99
    # exact verification emits the target's greedy continuation whatever tree the draft proposes
    same = (outs[True] == outs[False]).float().mean().item()
    assert same >= 0.95, same


def test_graphs_do_not_outlive_the_cache_they_were_captured_over():
    """Two generations with the same draft model over two caches: a graph captured over the first cache holds the
    addresses of its K / V rows and must not be replayed over the second; an eager speculation that needs a larger layer
    workspace in between must not pull the workspace from under a captured graph."""
    w = init_weights(CFG, 9, DEV)
    prompt = torch.randint(0, CFG.vocab_size, (1, 40), generator=torch.Generator().manual_seed(4)).to(DEV)

    def generate(gen, kv, n):
        wandb_logger.clear_log_data()
        out = gen.generate(prompt, max_new_tokens=n, do_sample=False, past_key_values=kv)[0].cpu()
        return out

    kv_ref = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv_ref, device=DEV, weights=w)
    plain = SubSpecSDGenerator(target, None, SubSpecSDDraftModel(draft), DraftParams(temperature=0.2, max_depth=4, topk_len=4),
                               generator_kwargs=dict(verify_method="exact", draft_graph=False))
    want = generate(plain, kv_ref, 40)

    kv1 = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    target, draft, _ = build_models(CFG, kv1, device=DEV, weights=w)
    dm = SubSpecSDDraftModel(draft)
    gen = SubSpecSDGenerator(target, None, dm, DraftParams(temperature=0.2, max_depth=4, topk_len=4),
                             generator_kwargs=dict(verify_method="exact", draft_graph=True))
    dm.graph_bucket = 32
    first = generate(gen, kv1, 40)
    assert dm.graph_replays > 0 and len(dm._graphs) >= 2
    held = len(dm._graphs)
    # a second cache: the graphs of the first are dropped, new ones are captured over the new storage
    kv2 = create_kv_cache("static", max_cache_len=512, config=CFG, device=DEV, dtype=torch.bfloat16)
    kv1.cache.data.fill_(float("nan"))                       # whatever still pointed at the old cache would show
    second = generate(gen, kv2, 40)
    assert all(e["cache_data"] is kv2.cache.data for e in dm._graphs.values())
    # an eager call that needs more workspace than any graph (a 64-row window) between two replays over the same cache
    kv2.reset()
    draft.tree_forward(torch.zeros(64, dtype=torch.long, device=DEV), torch.zeros(64, dtype=torch.long, device=DEV),
                       torch.ones(64, dtype=torch.int64, device=DEV), 100)
    torch.cuda.synchronize()
    kv2.reset()
    third = generate(gen, kv2, 40)
    for tag, got in (("first", first), ("second", second), ("third", third)):
        same = (got == want).float().mean().item()
        assert same >= 0.95, (tag, same)                     # exact verification: the target's tokens whatever the draft proposes
    assert torch.equal(second, third)
    # the number of captured buckets is bounded
    dm.max_graphs = 2
    dm._graphs.clear()
    kv2.reset()
    generate(gen, kv2, 60)
    assert len(dm._graphs) <= 2 and held >= 2
