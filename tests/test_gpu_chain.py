"""The denoise loop of the reference (fastdllm_engine.py:2133-2157: forward the block, shift, confidence, transfer
rule, until no mask token is left) run end to end through the library for a small stand-in model, captured once as a
HIP graph and replayed step by step, against the same chain on the oracle.

The stand-in model has two attention layers.  Per layer the active rows' q / k / v are table lookups of the
block's current token ids plus a position term (exact on both sides, so the K/V rows the library stores into the
block pages can be compared bit for bit); the attention of the active rows over [selected prefix pages || the block]
is the library's (GPU) or the oracle's (CPU).  The logits of a row come from a table row chosen by an integer hash of
the whole block's token ids (so every step's logits depend on every earlier decision) plus a small projection of the
two attention outputs.  The table is built with clear margins -- confident rows at 0.99, the others spaced in
confidence -- so that tokens, transfer decisions and the number of steps are fixed by the chain's logic, not by
rounding: they must agree exactly, the attention outputs within the attention bound."""
import math

import pytest
import torch

from oracle import ref_ops
from oracle.tolerances import assert_attn_close

pytestmark = pytest.mark.gpu

V, MASK, BLOCK, T_ROWS = 512, 511, 32, 64
HQ, HKV, D, P, LAYERS = 8, 2, 128, 256, 2
N_REQ, N_CHUNKS, TOPK, CHUNK = 2, 6, 3, 300
THRESHOLD = 0.9


def _model(seed):
    g = torch.Generator().manual_seed(seed)
    bf = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    m = {"q_tok": [bf(V, HQ, D) for _ in range(LAYERS)], "k_tok": [bf(V, HKV, D) for _ in range(LAYERS)],
         "v_tok": [bf(V, HKV, D) for _ in range(LAYERS)], "q_pos": [bf(BLOCK, HQ, D, std=0.5) for _ in range(LAYERS)],
         "k_pos": [bf(BLOCK, HKV, D, std=0.5) for _ in range(LAYERS)], "proj": torch.randn(HQ * D, V, generator=g) * 0.05}
    # logits table: row t is confident (one token 12 above the noise) or has a modest peak whose height is its own
    table = torch.randn(T_ROWS, V, generator=g) * 0.3
    flat_level = 0
    for t in range(T_ROWS):
        tok = int(torch.randint(0, V - 1, (1,), generator=g))
        if t % 3 == 0:
            table[t, tok] = 12.0
        else:
            table[t, tok] = 0.5 + 0.1 * flat_level      # confidences 0.003 .. 0.14, a level apart
            flat_level += 1
        table[t, MASK] = -10.0                          # the mask token is never sampled
    m["table"] = table.to(torch.bfloat16)
    m["last_logit"] = bf(N_REQ, V, std=0.3)
    m["hash_w"] = torch.arange(1, BLOCK + 1, dtype=torch.int64) * 7 + 3
    return m


def _prefix(seed):
    g = torch.Generator().manual_seed(seed)
    pages_per_req = (N_CHUNKS * CHUNK + P - 1) // P
    n_pages = N_REQ * pages_per_req + N_REQ          # + one block page per request
    kv = (torch.randn(2, LAYERS, n_pages, P, HKV, D, generator=g)).to(torch.bfloat16)
    perm = torch.randperm(n_pages - N_REQ, generator=g)
    block_table = torch.stack([perm[r * pages_per_req:(r + 1) * pages_per_req] for r in range(N_REQ)]).to(torch.int32)
    ranges = [[(c * CHUNK, CHUNK) for c in sorted(torch.randperm(N_CHUNKS, generator=g)[:TOPK].tolist())]
              for _ in range(N_REQ)]
    block_pages = torch.arange(n_pages - N_REQ, n_pages)
    slots = (block_pages.repeat_interleave(BLOCK) * P + torch.arange(BLOCK).repeat(N_REQ)).to(torch.int32)
    return kv, block_table, ranges, slots


def _rows(m, layer, ids):
    """q, k, v of the active rows: token tables + position terms (bf16 additions: the same bits on CPU and GPU)."""
    flat = ids.reshape(-1)
    pos = torch.arange(BLOCK, device=ids.device).repeat(ids.shape[0])
    return (m["q_tok"][layer][flat] + m["q_pos"][layer][pos], m["k_tok"][layer][flat] + m["k_pos"][layer][pos],
            m["v_tok"][layer][flat])


def _logits(m, ids, outs):
    """Table row (hash of the block's ids + 3 * position) % T_ROWS, plus a projection of the attention outputs that is
    too small to move a peak across a rounding boundary."""
    key = (ids * m["hash_w"].to(ids.device)).sum(dim=1)                                   # [n_req]
    t = (key[:, None] + 3 * torch.arange(BLOCK, device=ids.device)[None, :]) % T_ROWS     # distinct rows per request
    base = m["table"].to(ids.device)[t.reshape(-1)].float()
    feat = sum(o.float() for o in outs).reshape(-1, HQ * D) / LAYERS
    pert = 0.0005 * torch.tanh(feat @ m["proj"].to(ids.device))
    return (base + pert).to(torch.bfloat16)


def _oracle_chain(m, kv, block_table, ranges, slots):
    ids = torch.full((N_REQ, BLOCK), MASK, dtype=torch.int64)
    ids[:, 0] = torch.tensor([5, 77])
    qsl = [r * BLOCK for r in range(N_REQ + 1)]
    trace = []
    while bool((ids == MASK).any()):
        outs, stored = [], []
        for l in range(LAYERS):
            q, k, v = _rows(m, l, ids)
            ref_ops.store_kvcache(k, v, kv[0, l], kv[1, l], slots)
            outs.append(ref_ops.sparse_decode_attention(q, k, v, kv[0, l], kv[1, l], block_table, qsl, ranges))
            stored.append((k.clone(), v.clone()))
        logits = _logits(m, ids, outs)
        new_ids = ids.clone()
        for r in range(N_REQ):
            sl = slice(r * BLOCK, (r + 1) * BLOCK)
            conf, tok = ref_ops.sample_tokens(ref_ops.shift_logits(logits[sl], m["last_logit"][r]))
            new_ids[r], _ = ref_ops.threshold_unmask(ids[r], conf, tok, MASK, THRESHOLD)
        ids = new_ids
        trace.append((ids.clone(), outs, stored))
        assert len(trace) <= BLOCK
    return trace


def test_denoise_loop_as_replayed_graph_matches_oracle_chain(dev):
    from prefilling_dllm_amd import ops
    m = _model(3)
    kv, block_table, ranges, slots = _prefix(4)
    trace = _oracle_chain(m, kv.clone(), block_table, ranges, slots)
    assert 3 <= len(trace) <= BLOCK                     # several steps, some of them transferring more than one row

    md = {k: ([t.to(dev) for t in v] if isinstance(v, list) else v.to(dev)) for k, v in m.items()}
    dkv = kv.to(dev)
    ids = torch.full((N_REQ, BLOCK), MASK, dtype=torch.int64, device=dev)
    ids[:, 0] = torch.tensor([5, 77], device=dev)
    qsl = torch.arange(0, N_REQ * BLOCK + 1, BLOCK, dtype=torch.int32, device=dev)
    mk = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    ptr, start, length = [0], [], []
    for rr in ranges:
        start += [a for a, _ in rr]
        length += [b for _, b in rr]
        ptr.append(len(start))
    n = N_REQ * BLOCK
    qb = [torch.empty(n, HQ, D, dtype=torch.bfloat16, device=dev) for _ in range(LAYERS)]
    kb = [torch.empty(n, HKV, D, dtype=torch.bfloat16, device=dev) for _ in range(LAYERS)]
    vb = [torch.empty(n, HKV, D, dtype=torch.bfloat16, device=dev) for _ in range(LAYERS)]
    table = ops.new_slot_table(N_REQ, TOPK * CHUNK, dev)
    attn = [ops.PreparedAttention(qb[l], kb[l], vb[l], dkv[0, l], dkv[1, l], block_table.to(dev), qsl, max_q_len=BLOCK,
                                  max_ctx_len=TOPK * CHUNK, ranges=(mk(ptr), mk(start), mk(length), TOPK),
                                  slot_table=table, active_slot_mapping=slots.to(dev)) for l in range(LAYERS)]
    logits = torch.empty(n, V, dtype=torch.bfloat16, device=dev)
    unmask = ops.PreparedDenoiseUnmask(logits, ids, MASK, THRESHOLD, shift=True, last_logit=md["last_logit"])

    def step():
        attn[0].build_slot_table()
        for l in range(LAYERS):
            q, k, v = _rows(md, l, ids)
            qb[l].copy_(q); kb[l].copy_(k); vb[l].copy_(v)
            attn[l].run()
        logits.copy_(_logits(md, ids, [a.out for a in attn]))
        unmask.run()

    # eager warm-up on a scratch copy of the state, then capture one step and replay it
    saved_ids, saved_kv = ids.clone(), dkv.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ids.copy_(saved_ids); dkv.copy_(saved_kv)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    ids.copy_(saved_ids); dkv.copy_(saved_kv)
    torch.cuda.synchronize()

    steps = 0
    while True:
        graph.replay()
        left = unmask.left.cpu()                        # the loop's stop condition, read once per step
        ref_ids, ref_outs, ref_stored = trace[steps]
        assert torch.equal(ids.cpu(), ref_ids), f"step {steps}: block ids differ"
        for l in range(LAYERS):
            assert_attn_close(attn[l].out.float().cpu(), ref_outs[l], f"step {steps} layer {l}")
            # the block pages hold the rows this step stored (rewritten every step as ids change)
            got_k = dkv[0, l].view(-1, HKV, D)[slots.to(dev).long()].cpu()
            got_v = dkv[1, l].view(-1, HKV, D)[slots.to(dev).long()].cpu()
            assert torch.equal(got_k, ref_stored[l][0]) and torch.equal(got_v, ref_stored[l][1])
        assert left.tolist() == [int((ref_ids[r] == MASK).sum()) for r in range(N_REQ)]
        steps += 1
        if int(left.sum()) == 0:
            break
        assert steps < len(trace), "the library's loop runs longer than the oracle's"
    assert steps == len(trace)
