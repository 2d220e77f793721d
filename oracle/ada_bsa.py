"""Oracle: adaptive block-sparse attention on the CPU (test infrastructure only).

Restates the numpy statements the reference's tests hold for its two in-tree AscendC kernels:
``sparse_estimate`` follows tests/plugin/test_sparseblockestimate.py:24-36 (softmax_flash) and :49-145
(sparse_estimate_cpu), ``ada_block_sparse_attention`` follows
tests/plugin/test_adablocksparseattention.py:35-87.  The reference's test exercises the non-causal estimate only
(test_sparseblockestimate.py:166); the causal branches of its numpy statement are restated as they stand.  Its
own tolerance for the estimate is a mask difference below 2 % of the selected blocks and fewer than 1 % omitted
blocks (:231-241).  The selection exists twice in the reference: as that numpy statement (``select_blocks``) and as
the kernel's ScoreCompute (csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h:947-1078, restated as
``select_blocks_kernel``); they differ in how the first block and the switches are treated, and the product
follows the kernel.
"""
import numpy as np
import torch

M_ROWS, N_COLS = 128, 1024  # strided rows / columns per step of the reference's loops (:56)


def softmax_flash(src, inmax=None, insum=None):
    """One step of the running softmax (:24-36): exp against the maximum seen so far, running sum."""
    if inmax is None:
        x_max = src.max(axis=-1, keepdims=True)
        dst = np.exp(src - x_max)
        return dst, x_max, dst.sum(axis=-1, keepdims=True)
    x_max = np.maximum(inmax, src.max(axis=-1, keepdims=True))
    dst = np.exp(src - x_max)
    return dst, x_max, np.exp(inmax - x_max) * insum + dst.sum(axis=-1, keepdims=True)


def _pad_rows(x, multiple):
    r = x.shape[0] % multiple
    return x if r == 0 else np.concatenate([x, np.zeros((multiple - r,) + x.shape[1:], dtype=x.dtype)], axis=0)


def strided_scores(q, k, stride=8):
    """[Sq, D] x [Sk, D] -> anti-diagonal strided scores [ceil(Sq/stride), ceil(Sk/stride)] (:65-69, :84, :86):
    P'[i][j] = sum_s q[stride*i + stride-1-s] . k[stride*j + s] / (sqrt(D) * stride), tokens past S are zeros."""
    d = q.shape[-1]
    qs = _pad_rows(q.astype(np.float32), stride).reshape(-1, stride, d)[:, ::-1, :].reshape(-1, stride * d)
    ks = _pad_rows(k.astype(np.float32), stride).reshape(-1, stride * d)
    return np.dot(qs / (np.sqrt(d) * stride), ks.T)


def block_scores(q, k, blocksize=128, stride=8, causal=False):
    """Share of the estimated attention mass per (query block, key block), with the reference's loop
    structure: 128 strided rows at a time, columns in steps of 1024 with a running softmax, first reduction
    over groups of blocksize/stride columns, rescaling to the final maximum and sum, second reduction over
    groups of rows (:58-119).  ``causal``: a step of 1024 query tokens sees the keys up to its own end, cut
    down to whole groups of ``stride`` tokens (:71, :78); the result then has a row of blocks per query
    block but only as many columns as the last step saw, earlier rows are zero padded."""
    reduce_size = blocksize // stride
    seq = q.shape[0]
    nb = (seq + blocksize - 1) // blocksize
    out = []
    for r0 in range(0, seq, M_ROWS * stride):
        qc = q[r0:r0 + M_ROWS * stride]
        kseq = seq if not causal else (r0 + qc.shape[0]) // stride * stride
        first, maxes, x_max, x_sum = [], [], None, None
        for c0 in range(0, kseq, N_COLS * stride):
            p = strided_scores(qc, k[c0:min(kseq, c0 + N_COLS * stride)], stride)
            p, x_max, x_sum = softmax_flash(p, x_max, x_sum)
            pc = p.shape[1] % reduce_size
            if pc:
                p = np.concatenate([p, np.zeros((p.shape[0], reduce_size - pc), dtype=np.float32)], axis=1)
            first.append(p.reshape(p.shape[0], -1, reduce_size).sum(axis=-1))
            maxes.append(x_max.copy())
        rows = []
        for part, mx in zip(first, maxes):
            part = _pad_rows(part * (np.exp(mx - x_max) / x_sum), reduce_size)
            rows.append(part.reshape(-1, reduce_size, part.shape[1]).sum(axis=1))
        blk = np.concatenate(rows, axis=-1)
        if blk.shape[1] < nb:
            blk = np.concatenate([blk, np.zeros((blk.shape[0], nb - blk.shape[1]), dtype=blk.dtype)], axis=1)
        out.append(blk[:, :max(nb, blk.shape[1])])
    return np.concatenate(out, axis=0)


def select_blocks(score_row, threshold, force_sparse, keep_sink=True, keep_recent=True):
    """One row of block scores -> boolean selection (:126-143, non-causal): the last block is left out of
    the ranking; blocks in descending order are counted until the running sum reaches threshold * total;
    the count is capped at force_sparse * blocks; the first and the last block are forced (the numpy
    statement always forces both; the switches are the kernel's setFirst / setDiag,
    csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h:1044-1049)."""
    to_sort = np.array(score_row, dtype=np.float32).copy()
    to_sort[-1] = 0
    score = -np.sort(-to_sort, kind="stable").astype(np.float32)
    cnt = int((score.cumsum() < threshold * score.sum()).astype(np.int32).sum()) + 1
    if force_sparse > 0 and cnt > force_sparse * score.shape[-1]:
        cnt = int(force_sparse * score.shape[-1])
    cnt = max(1, min(cnt, score.shape[-1]))
    guard = score[cnt - 1]
    if keep_sink:
        to_sort[0] = guard + 1
    if keep_recent:
        to_sort[-1] = guard + 1
    return to_sort >= guard


SBE_EPS = 1e-5  # sparse_block_estimate.h:85


def select_blocks_kernel(score_row, threshold, row_sparse, keep_sink=True, keep_recent=True, causal=False):
    """The reference kernel's selection for one row (ScoreCompute, sparse_block_estimate.h:947-1078);
    ``score_row`` holds the columns that take part (all blocks, or with ``causal`` those up to the diagonal).
    Differences from ``select_blocks``: the first block is left out of the ranking and of the total when
    ``keep_sink`` (setFirst) is set and is kept in any case (:1067); without ``causal`` the last block is left
    out and forced whatever ``keep_recent`` (setDiag) says (:976-978, :1051-1053); the cap only applies from 10
    columns on (:1046); a threshold >= 1 keeps every column (:1042-1045); the guard is lowered by 1e-5 (:1047)."""
    src = np.array(score_row, dtype=np.float32).copy()
    n = src.shape[0]
    if causal and n <= 2:                                    # :958-962
        return np.ones(n, dtype=np.bool_)
    last_out = keep_recent or not causal
    if last_out:                                             # :976-978: the mask of ranked columns stops before it
        src[-1] = 0
    if keep_sink:                                            # :980-983
        src[0] = 0
    ranked = -np.sort(-src, kind="stable")                   # :996
    if threshold < 1.0:                                      # :1009-1041: first column at which the running sum
        run = np.cumsum(ranked, dtype=np.float32)            # reaches threshold * total (:991 total of the ranked ones)
        hit = np.nonzero(run >= np.float32(threshold) * run[-1])[0]
        cnt = int(hit[0]) if hit.size else n - 1
        guard = np.float32(ranked[cnt])
    else:                                                    # :1042-1045
        cnt, guard = n, np.float32(0.0)
    if cnt > n * row_sparse and n >= 10:                     # :1046-1049
        guard = np.float32(ranked[max(int(n * row_sparse), 1) - 1])
    guard = np.float32(guard - np.float32(SBE_EPS))          # :1047
    if keep_sink:                                            # :1048-1050
        src[0] = guard + 1
    if last_out:                                             # :1051-1053
        src[-1] = guard + 1
    keep = src > guard                                       # :1056-1066: relu(x - guard) / (relu + 0.001), rounded up
    keep[0] = True                                           # :1067
    return keep


def sparse_estimate(query, key, blocksize=128, stride=8, threshold=0.5, force_sparse=1.0, keep_sink=True,
                    keep_recent=True, causal=False, rules="numpy"):
    """[B, N, S, D] query / key (any float dtype) -> boolean mask [B, N, nb, nb], nb = ceil(S / blocksize).
    ``rules``: 'numpy' = the selection of the reference's numpy statement, 'kernel' = that of its kernel.
    ``causal`` (:121-127, :140): row i selects among its first i + 1 blocks, the diagonal block standing where
    the last block stands otherwise (forced only with ``keep_recent``, the kernel's setDiag,
    sparse_block_estimate.h:1047-1049); rows 0 and 1 keep their whole prefix."""
    bs, nq, seq, _ = query.shape
    gqa = nq // key.shape[1]
    nb = (seq + blocksize - 1) // blocksize
    mask = np.zeros((bs, nq, nb, nb), dtype=np.bool_)
    qf, kf = query.float().numpy(), key.float().numpy()
    for bi in range(bs):
        for ni in range(nq):
            sc = block_scores(qf[bi, ni], kf[bi, ni // gqa], blocksize, stride, causal)
            for i in range(nb):
                n = i + 1 if causal else nb
                if rules == "kernel":
                    mask[bi, ni, i, :n] = select_blocks_kernel(sc[i, :n], threshold, force_sparse, keep_sink,
                                                               keep_recent, causal)
                elif causal and i <= 1:
                    mask[bi, ni, i, :n] = True
                else:
                    mask[bi, ni, i, :n] = select_blocks(sc[i, :n], threshold, force_sparse, keep_sink, keep_recent)
    return mask


def ada_block_sparse_attention(query, key, value, smask, causal=False, blocksize=128, rules="numpy"):
    """test_adablocksparseattention.py:35-87: every query block attends to the keys of the blocks its mask row
    selects; with ``causal`` the upper triangle of the last ``t`` gathered keys (``t`` = rows of the query
    block) gets -10000 added, i.e. the last selected block is taken to be the diagonal block.
    ``rules="kernel"``: the reference kernel applies that triangle only when the last selected block IS the
    diagonal block (``isLastBlockCausalDiag``, ada_block_sparse_attention_s1s2_bns1_x910.h:245-259, :512-514);
    the two statements agree on every mask whose rows end with their diagonal block (what the estimate
    produces with ``keep_recent``)."""
    bs, nq, seq, dim = query.shape
    gqa = nq // key.shape[1]
    out = torch.zeros(bs, nq, seq, dim, dtype=torch.float32)
    qf, kf, vf = query.float().numpy(), key.float().numpy(), value.float().numpy()
    sm = np.asarray(smask).astype(bool)
    nb = (seq + blocksize - 1) // blocksize
    for bi in range(bs):
        for ni in range(nq):
            for s1 in range(nb):
                sel = np.repeat(sm[bi, ni, s1, :nb], blocksize)[:seq]
                start, end = s1 * blocksize, min((s1 + 1) * blocksize, seq)
                k = kf[bi, ni // gqa][sel]
                if k.shape[0] == 0:
                    continue
                p = qf[bi, ni, start:end] @ k.T / np.sqrt(dim)
                if causal and (rules == "numpy" or np.flatnonzero(sm[bi, ni, s1, :nb])[-1] == s1):
                    t = end - start
                    p[:, -t:] += np.triu(np.ones((t, t)), k=1) * (-10000.0)
                p = p - p.max(axis=-1, keepdims=True)
                e = np.exp(p)
                out[bi, ni, start:end] = torch.from_numpy((e / (e.sum(axis=-1, keepdims=True) + 1e-12)) @ vf[bi, ni // gqa][sel])
    return out
