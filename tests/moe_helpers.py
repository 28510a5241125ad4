"""Routing tables for the MoE dispatch/combine tests and the benchmark: per rank, router logits
N(0,1) from the (seed, rank) generator, top-k experts per token (ties to the lower expert id),
expert e owned by rank e // experts_per_rank, (token, expert) pairs sorted by (expert, token)."""
import numpy as np
import torch


def route(n, tokens, n_experts, topk, seed=1234):
    per_rank = n_experts // n
    S = np.zeros((n, n), dtype=np.int64)
    send_tok, send_exp = [], []
    for r in range(n):
        g = torch.Generator().manual_seed(seed * 1_000_003 + r)
        logits = torch.randn(tokens, n_experts, generator=g)
        experts = torch.topk(logits, topk, dim=1).indices
        tok = torch.arange(tokens).repeat_interleave(topk)
        exp = experts.reshape(-1)
        order = torch.argsort(exp * tokens + tok, stable=True)
        send_tok.append(tok[order].contiguous())            # source row of every sent row, in send order
        send_exp.append(exp[order].contiguous())
        S[r] = np.bincount((exp[order] // per_rank).numpy(), minlength=n)
    return S, send_tok, send_exp


def combine_tables(n, tokens, topk, S, send_tok):
    """Where each (token, k) copy of rank r ended up after the dispatch: (destination rank, row in
    that rank's receive buffer).  k enumerates a token's copies in send order."""
    src_rank, src_row = [], []
    recv_base = np.zeros((n, n), dtype=np.int64)            # recv_base[r][d]: row offset of segment r in d's buffer
    for d in range(n):
        recv_base[:, d] = np.concatenate([[0], np.cumsum(S[:-1, d])])
    for r in range(n):
        dest = np.repeat(np.arange(n), S[r])                # destination of every sent row
        within = np.concatenate([np.arange(c) for c in S[r]]) if S[r].sum() else np.zeros(0, dtype=np.int64)
        row = recv_base[r][dest] + within
        tok = send_tok[r].numpy()
        order = np.argsort(tok, kind="stable")               # group a token's copies together
        src_rank.append(torch.from_numpy(dest[order].astype(np.int32)).view(tokens, topk).contiguous())
        src_row.append(torch.from_numpy(row[order].astype(np.int64)).view(tokens, topk).contiguous())
    return src_rank, src_row
