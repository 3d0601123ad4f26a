"""Vedadra test bodies, parametrised by device and dtype: the CPU file runs them on the
framework's PyTorch ops in fp32, the GPU file on the HIP kernels in fp32 and bf16."""

from __future__ import annotations

import numpy as np
import torch

import vedadra_common as C
from oracles import vedadra_oracle as O


def tol(dtype):
    # fp32 is the sharp check; bf16 activations round at every product of these tiny models
    return 2e-4 if dtype == torch.float32 else 0.12


def ktol(dtype):
    """Kernel-level checks: inputs are already rounded to the dtype, so only the kernel's own
    roundings (bf16 outputs) remain."""
    return 2e-4 if dtype == torch.float32 else 1.5e-2


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _check(got, want, dtype, what):
    e = C.rel_err(got, want)
    assert e < tol(dtype), (what, e)


def _np(t):
    return t.double().cpu().numpy()


# ------------------------------------------------------------------ mechanisms alone
def case_group_norm(device, dtype):
    """Every combination of the sublayer-boundary step: output norm + residual, added rows,
    next input norm; group counts 1, 3, 4 and one group per pair of columns; the sublayer output
    as a stored row (use_y 1) or as the split-K partial sums of its GEMM plus a bias (use_y 2)."""
    from enterprise_inference_amd.ops import norm
    from enterprise_inference_amd.ops.gemm import SplitK
    g = torch.Generator().manual_seed(1)
    for W, groups in ((48, 3), (40, 1), (256, 4), (64, 32), (130, 2)):
        for use_y, use_add, use_next in ((1, 0, 1), (1, 1, 1), (0, 0, 1), (0, 1, 1), (1, 0, 0),
                                         (2, 0, 1), (2, 1, 0)):
            x = torch.randn(5, W, generator=g) * 2
            y = (torch.randn(5, W, generator=g) * 3 + 0.5).to(dtype)
            part = torch.randn(3, 5, W, generator=g) * 2
            bias = torch.randn(W, generator=g).to(dtype)
            if use_y == 2:
                y = part.double().sum(0) + bias.double()
            add = torch.randn(5, W, generator=g)
            w1 = torch.randn(W, generator=g).to(dtype)
            w2 = torch.randn(W, generator=g).to(dtype)
            want_x, want_h = [], []
            for r in range(5):
                v = _np(x[r])
                if use_y:
                    v = v + O.group_norm(_np(y[r]), _np(w1), groups, 1e-5)
                if use_add:
                    v = v + _np(add[r])
                want_x.append(v)
                want_h.append(O.group_norm(v, _np(w2), groups, 1e-5))
            xd = x.clone().to(device)
            if use_y == 2:
                y_in = SplitK(part.to(device), 3, 5, W, bias.to(device))
            else:
                y_in = y.to(device) if use_y else None
            h = norm.group_norm_step(xd, groups, 1e-5, y_in,
                                     w1.to(device) if use_y else None,
                                     add.to(device) if use_add else None,
                                     w2.to(device) if use_next else None)
            assert np.allclose(_np(xd), np.stack(want_x), atol=2e-5, rtol=1e-5), (W, groups)
            if use_next:
                assert h.dtype == dtype
                assert np.allclose(_np(h), np.stack(want_h), atol=ktol(dtype), rtol=ktol(dtype))
            else:
                assert h is None


def case_qk_norm_cache(device, dtype):
    """Per-map RMS norm of queries and keys, values copied as projected (also when they are the
    un-normed key columns), rows without a slot skipped, other slots untouched."""
    from enterprise_inference_amd.ops import window_attention as wa
    from enterprise_inference_amd.ops.gemm import SplitK
    g = torch.Generator().manual_seed(2)
    for mq, mk, D, vw, alias, split in ((4, 2, 16, 32, True, 0), (6, 2, 10, 14, False, 0),
                                        (2, 2, 96, 40, False, 0), (1, 1, 5, 5, True, 0),
                                        (4, 2, 16, 32, True, 3), (3, 1, 24, 20, False, 2)):
        T, bs, nb = 7, 4, 5
        k_off, q_off = 3, 3 + mk * D + (0 if alias else vw)
        v_off = k_off if alias else k_off + mk * D
        width = q_off + mq * D + 2
        fused = (torch.randn(T, width, generator=g) * 2).to(dtype)
        part = torch.randn(max(split, 1), T, width, generator=g)
        bias = torch.randn(width, generator=g).to(dtype)
        qw = (1 + 0.3 * torch.randn(D, generator=g)).to(dtype)
        kw = (1 + 0.3 * torch.randn(D, generator=g)).to(dtype)
        slots = torch.tensor([9, 2, -1, 17, 0, 5, 19], dtype=torch.int32)
        kc = torch.full((nb, bs, mk * D), 7.0, dtype=dtype)
        vc = torch.full((nb, vw, bs), 7.0, dtype=dtype)
        kd, vd = kc.to(device), vc.to(device)
        src = SplitK(part.to(device), split, T, width, bias.to(device)) if split else fused.to(device)
        q, gate = wa.qk_norm_cache(src, q_off, k_off, v_off, mq, mk, D, vw, qw.to(device),
                                   kw.to(device), kd, vd, slots.to(device), 1e-5, 1, 3)
        f = (part.double().sum(0) + bias.double()).numpy() if split else _np(fused)
        assert np.allclose(_np(gate), f[:, 1:4], atol=ktol(dtype), rtol=ktol(dtype))
        for t in range(T):
            for m in range(mq):
                want = O.rms_div(f[t, q_off + m * D:q_off + (m + 1) * D], 1e-5) * _np(qw)
                assert np.allclose(_np(q[t, m * D:(m + 1) * D]), want, atol=ktol(dtype), rtol=ktol(dtype))
        kflat = _np(kd).reshape(nb * bs, -1)
        vflat = _np(vd.permute(0, 2, 1)).reshape(nb * bs, -1)
        used = set()
        for t, s in enumerate(slots.tolist()):
            if s < 0:
                continue
            used.add(s)
            for m in range(mk):
                want = O.rms_div(f[t, k_off + m * D:k_off + (m + 1) * D], 1e-5) * _np(kw)
                assert np.allclose(kflat[s, m * D:(m + 1) * D], want, atol=ktol(dtype), rtol=ktol(dtype))
            assert np.allclose(vflat[s], f[t, v_off:v_off + vw], atol=ktol(dtype) if split else 0,
                               rtol=ktol(dtype) if split else 0)
        for s in range(nb * bs):
            if s not in used:
                assert (kflat[s] == 7.0).all() and (vflat[s] == 7.0).all()


def _paged(n, bs, seed):
    """A shuffled block table for n tokens and the slot of every position."""
    nblk = -(-n // bs)
    g = torch.Generator().manual_seed(seed)
    table = (torch.randperm(nblk + 3, generator=g)[:nblk]).to(torch.int32)
    slots = torch.tensor([int(table[j // bs]) * bs + j % bs for j in range(n)])
    return table, slots, nblk + 3


def _metadata(device, table, decode_pos, chunk):
    """One sequence seen as decode rows (one per position in decode_pos, every row its own copy
    of the sequence) followed by one prefill chunk (start, n)."""
    from enterprise_inference_amd.ops.attention import AttentionMetadata
    nd = len(decode_pos)
    start, n = chunk
    pos = torch.tensor(list(decode_pos) + list(range(start, start + n)), dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return AttentionMetadata(
        num_decode=nd, num_prefill_tokens=n,
        slot_mapping=torch.full((nd + n,), -1, dtype=torch.int32, device=device),
        positions=pos.to(device),
        decode_block_tables=table[None, :].repeat(max(nd, 1), 1).contiguous().to(device),
        decode_seq_lens=i32([p + 1 for p in decode_pos]) if nd else None,
        prefill_block_tables=table[None, :].contiguous().to(device) if n else None,
        prefill_seq_lens=i32([start + n]) if n else None,
        prefill_cu_q=i32([0, n]) if n else None, prefill_q_lens=[n] if n else None)


def case_window_needle(device, dtype, kind="talking", H=4, G=2, D=16, Dv=16, size=40, keep=0,
                       n=150, bs=16):
    """One key made to stand out: the query at position i and the key at position j share a large
    component, so the output is that key's value when j is visible and far from it when not.
    j runs over the window's inside and outside edge, the kept first tokens and the token after
    them, page borders and far keys; i is read as a prefill row and as a decode row."""
    from enterprise_inference_amd.ops import window_attention as wa
    P = 1 if kind == "talking" else 2
    if kind == "talking":
        Dv = D
    g = torch.Generator().manual_seed(3)
    table, slots, nblk = _paged(n, bs, 4)
    i = n - 7
    edge = i - size + 1
    cand = {edge, edge - 1, edge + 1, i, i - 1, 0, n // 3, edge - 40,
            (edge // bs) * bs, (edge // bs) * bs - 1, (i // bs) * bs, (i // bs) * bs - 1}
    if keep:
        cand |= {keep - 1, keep, keep + 1}
    temp = (1 + 0.3 * torch.randn(H, generator=g)).abs() + 0.2
    talk = torch.eye(H) + 0.2 * torch.randn(H, H, generator=g)
    spec = wa.WindowSpec(H, G, P, D, Dv, size, keep, mult=(temp * 0.3 if kind == "talking" else
                                                            torch.full((H * P,), 0.3)).to(device))
    lam, diff = 0.37, 0.2
    if kind == "talking":
        hh = torch.arange(1, H + 1, dtype=torch.float64)
        spec.slope = torch.pow(2.0, -8.0 * hh / H).float().to(device)
        spec.talk = talk.to(device)
    else:
        spec.epilogue, spec.eps, spec.post = 1, 1e-5, 1.0 - diff
        spec.lam = torch.tensor([lam], dtype=torch.float32, device=device)
    for j in sorted(c for c in cand if 0 <= c <= i):
        q = torch.randn(n, H * P, D, generator=g) * 0.5
        k = torch.randn(n, G * P, D, generator=g) * 0.5
        v = torch.randn(n, G, Dv, generator=g)
        gate = torch.randn(n, H * Dv, generator=g)
        u = torch.zeros(D)
        u[j % D] = 1.0
        q[i] += 12.0 * u                       # every map of query i ...
        k[j] += 12.0 * u                       # ... meets every key map of token j
        q, k, v, gate = q.to(dtype), k.to(dtype), v.to(dtype), gate.to(dtype)
        kc = torch.zeros(nblk, bs, G * P * D, dtype=dtype)
        vc = torch.zeros(nblk, G * Dv, bs, dtype=dtype)
        kc.view(-1, G * P * D)[slots] = k.reshape(n, -1)
        vc[slots // bs, :, slots % bs] = v.reshape(n, -1)
        rows = [i, min(i + 3, n - 1), j]                          # decode rows ...
        chunk = (i - 5, 9)                                        # ... and a chunk around i
        md = _metadata(device, table, rows, chunk)
        pos = rows + list(range(chunk[0], chunk[0] + chunk[1]))
        qs = torch.stack([q[p].reshape(-1) for p in pos])
        gs = torch.stack([gate[p] for p in pos])
        got = wa.window_attention(qs.to(device), kc.to(device), vc.to(device), md, spec,
                                  gs.to(device) if kind == "talking" else None)
        kn = [_np(k[t]).reshape(G, P, D) if P == 2 else _np(k[t]) for t in range(n)]
        vals = [_np(v[t]) for t in range(n)]
        for r, p in enumerate(pos):
            if kind == "talking":
                want = O.talking_heads(_np(q[p]), kn, vals, p, H, G, size, 0.3, _np(temp), _np(talk))
                want = want / (1.0 + np.exp(-_np(gate[p])))
            else:
                want = O.differential_heads(_np(q[p]).reshape(H, 2, D), kn, vals, p, H, G, size,
                                            keep, 0.3, lam, diff, 1e-5)
            d = np.abs(_np(got[r]) - want).max()
            assert d < (1e-4 if dtype == torch.float32 else 4e-2), (kind, j, p, d)


# ------------------------------------------------------------------ whole models
def case_layers(device, dtype, cfg_fn=C.config_a):
    """The residual stream after every layer run (a looped layer once per pass)."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, 9, dtype)
    t = _tokens(21, cfg["vocab"], 5)
    want = []
    C.oracle_logits(cfg, W, t, want)
    sess = C.make_session(cfg, W, device, dtype, max_tokens=64, block_size=16, max_live=1)
    try:
        from enterprise_inference_amd.engine.sequence import Sequence
        seq = Sequence("s", list(t), sess._params)
        plan = sess.scheduler.plan_given([(seq, len(t))])
        r = sess.runner
        r._flip_staging()
        sp = r._prepare_eager(sess.scheduler.bm, plan, logit_rows=[])
        r.d_e_buf[:sp["off"]].copy_(r.e_buf[:sp["off"]])
        ids, md, _ = r._eager_inputs(sp)
        got = []
        with torch.no_grad():
            r.model(ids, md, r.kv_caches, collect=got)
        r.finish_step()
        assert len(got) == len(want) == len(O.run_order(cfg))
        for k, (a, b) in enumerate(zip(got, want)):
            e = np.abs(_np(a) - b).max() / np.abs(b).max()
            assert e < (1e-4 if dtype == torch.float32 else 0.08), (k, e)
    finally:
        sess.close()


def case_schedules(device, dtype, cfg_fn=C.config_a, seed=0, block_size=16):
    """Whole prompts, prompt + one-by-one decoding, portions of several sizes down to two tokens
    and mixed batches with reuse of pages all give the oracle's logits."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, seed, dtype)
    V = cfg["vocab"]
    reqs = {"a": _tokens(70, V, 11), "b": _tokens(37, V, 12), "c": _tokens(5, V, 13),
            "d": _tokens(1, V, 14), "e": _tokens(49, V, 15)}
    want = {k: C.oracle_logits(cfg, W, t) for k, t in reqs.items()}
    # pool of 8 pages (of 16 tokens: "a" alone needs 5), so pages must be used again
    sess = C.make_session(cfg, W, device, dtype, max_tokens=8 * block_size, block_size=block_size,
                          max_live=2)
    try:
        for k, t in reqs.items():
            got = sess.step([{"id": k, "tokens": t, "want": list(range(len(t)))}], end=[k])
            _check(got, want[k], dtype, ("whole", k))
        # a prompt portion, then token by token: the windows pass over decoded tokens
        for k in ("a", "b"):
            t = reqs[k]
            n0 = len(t) - 34
            got = [sess.step([{"id": k, "tokens": t[:n0], "want": [n0 - 1]}])]
            for i in range(n0, len(t)):
                got.append(sess.step([{"id": k, "tokens": [t[i]], "want": [0]}],
                                     end=[k] if i == len(t) - 1 else []))
            _check(torch.cat(got), want[k][n0 - 1:], dtype, ("decode", k))
        # portions: sizes cross page borders (16) and window edges and go down to two tokens
        t, at, got = reqs["a"], 0, []
        for n in (2, 13, 2, 16, 1, 17, 2, 15, 2):
            got.append(sess.step([{"id": "a", "tokens": t[at:at + n], "want": list(range(n))}],
                                 end=["a"] if at + n == len(t) else []))
            at += n
        assert at == len(t)
        _check(torch.cat(got), want["a"], dtype, "portions")
    finally:
        sess.close()
    # mixed batches on 4 sequences / 10 pages: unequal requests side by side, decode rows beside
    # prompt portions, requests that pause, pages freed and taken again
    sess = C.make_session(cfg, W, device, dtype, max_tokens=10 * block_size, block_size=block_size,
                          max_live=4)
    try:
        got = {k: [] for k in reqs}
        at = {k: 0 for k in reqs}

        def run(plan, end=()):
            entries = []
            for k, n in plan:
                entries.append({"id": k, "tokens": reqs[k][at[k]:at[k] + n], "want": list(range(n))})
            out = sess.step(entries, end)
            r = 0
            for k, n in plan:
                got[k].append(out[r:r + n])
                r += n
                at[k] += n
        run([("d", 1), ("b", 3), ("c", 2)], end=["d"])
        run([("b", 1), ("c", 3), ("a", 20)], end=["c"])           # c finishes: its page is free
        run([("a", 1), ("e", 30), ("b", 17)])                     # e takes the freed pages
        run([("e", 1), ("b", 16), ("a", 2)], end=["b"])
        run([("a", 47)], end=["a"])                               # e pauses
        run([("e", 18)], end=["e"])
        for k in reqs:
            assert at[k] == len(reqs[k])
            _check(torch.cat(got[k]), want[k], dtype, ("mixed", k))
        # a second life for a finished request's name, on reused pages
        got2 = sess.step([{"id": "b", "tokens": reqs["b"], "want": list(range(len(reqs["b"])))},
                          {"id": "c", "tokens": reqs["c"], "want": [4]}], end=["b", "c"])
        _check(got2[:-1], want["b"], dtype, "again b")
        _check(got2[-1:], want["c"][4:], dtype, "again c")
        bm = sess.scheduler.bm
        assert bm.num_free_blocks() == bm.num_blocks
    finally:
        sess.close()


def case_long_decode(device, dtype, cfg_fn=C.config_b):
    """140 tokens decoded one by one after a 3-token prompt, over many page borders and far past
    every window."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, 3, dtype)
    t = _tokens(143, cfg["vocab"], 21)
    want = C.oracle_logits(cfg, W, t)
    sess = C.make_session(cfg, W, device, dtype, max_tokens=160, block_size=16, max_live=1)
    try:
        got = [sess.step([{"id": "x", "tokens": t[:3], "want": [0, 1, 2]}])]
        for i in range(3, len(t)):
            got.append(sess.step([{"id": "x", "tokens": [t[i]], "want": [0]}]))
        _check(torch.cat(got), want, dtype, "long decode")
    finally:
        sess.close()


def case_generate(device, dtype, cfg_fn=C.config_a, expect_graphs=None):
    """Greedy generation through LLMEngine (its scheduler, batching and sampler): every emitted
    token is the oracle's argmax given the tokens before it, for unequal prompts in one batch."""
    import copy

    from enterprise_inference_amd.config import (CacheConfig, EngineConfig, ModelConfig,
                                                 SchedulerConfig)
    from enterprise_inference_amd.engine.llm_engine import LLMEngine
    from enterprise_inference_amd.engine.sampling_params import SamplingParams
    cfg = cfg_fn()
    W = C.random_weights(cfg, 5, dtype)
    ec = EngineConfig(model=ModelConfig.from_hf_dict(copy.deepcopy(cfg)), dtype=dtype, device=device,
                      load_format="dummy",
                      cache=CacheConfig(block_size=16, num_gpu_blocks=24),
                      scheduler=SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=32,
                                                max_model_len=128))
    eng = LLMEngine(ec)
    model = eng.executor.runner.model
    model.load_weights(W.items())
    model.post_load()
    if expect_graphs is not None:
        assert bool(eng.executor.runner.graphs) == expect_graphs
    prompts = [_tokens(n, cfg["vocab"], 30 + n) for n in (40, 7, 1, 19)]     # 4 prompts, 3 seats
    outs = eng.generate(prompt_token_ids=prompts,
                        params=SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        toks = list(o.outputs[0].token_ids)
        assert len(toks) == 12
        lg = C.oracle_logits(cfg, W, p + toks[:-1])
        for i, tk in enumerate(toks):
            row = lg[len(p) - 1 + i]
            # the chosen token is the oracle's best, or within rounding of it
            assert float(row.max() - row[tk]) <= (1e-3 if dtype == torch.float32 else 0.15), (i, tk)
    eng.shutdown()
