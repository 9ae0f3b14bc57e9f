"""AutoFocusFormer classifier assembled around the CLUSTEN operators.

This is the build's own counterpart of models/aff_transformer.py, kept to what drives the three operators and
what an end-to-end images/s figure needs.  Parameter names and shapes equal the reference's, so a reference
`state_dict` loads unchanged.  What each class must reproduce:

  ClusterAttention  (aff_transformer.py:87-160)  q scaled by head_dim^-0.5 before QK; q/key/v handed to the
                    operators as permuted views of the Linear outputs; position bias, padding mask (-100),
                    blank token and softmax between QK and AV; dense branch when a stage attends globally.
  ClusterMerging    (aff_transformer.py:276-365) merge centres = top scores of grid prior + alpha * learned
                    score, reserve tokens on the coarse grid; weights (b, n', m, 4) = weight_net(table)[pe_idx] *
                    learned score * mask; WF output (b, n', 4, c) flattened so that channel = ic * c + c'.
  BasicLayer        (aff_transformer.py:441-507) balanced clusters, the nnc nearest clusters of every token, the
                    neighbourhood list = members of those clusters, nearest cluster first.

Differences from the reference, none of which change results: the relative-position table is a module buffer
instead of a module-level global; the neighbourhoods of the first stage, whose tokens sit on the image grid,
are computed once and reused (the reference caches the clustering but repeats the neighbour search); nearest
neighbours use a sort of exact distances instead of an external library; the operators are reached through
`self.ops`, so a test can run the very same modules on another implementation of the three functions.
"""
import math
from types import SimpleNamespace

import torch
import torch.nn as nn
import torch.nn.functional as F

from .points import knn, space_filling_cluster


def default_ops():
    """The three operators as the HIP library provides them."""
    from clusten import CLUSTENAVFunction, CLUSTENQKFunction, CLUSTENWFFunction, _native
    return SimpleNamespace(qk=CLUSTENQKFunction.apply, av=CLUSTENAVFunction.apply, wf=CLUSTENWFFunction.apply,
                           attn_softmax=_native.attn_softmax, attn_softmax_supported=_native.attn_softmax_supported,
                           qk_clusters=_native.qk_forward_clusters, av_clusters=_native.av_forward_clusters,
                           clusters_supported=_native.clusters_supported,
                           cluster_attention=_native.cluster_attention,
                           cluster_attention_plan=_native.cluster_attention_plan,
                           cluster_attention_supported=_native.cluster_attention_supported,
                           cluster_attention_backward=_native.cluster_attention_backward,
                           cluster_attention_backward_supported=_native.cluster_attention_backward_supported,
                           cluster_pairs=_native.cluster_pairs, scatter_rows=_native.scatter_rows,
                           dense_attention=_native.dense_attention,
                           dense_attention_supported=_native.dense_attention_supported,
                           layer_norm=_native.layer_norm, layer_norm_supported=_native.layer_norm_supported,
                           linear=_native.linear, linear_supported=_native.linear_supported,
                           add_layer_norm=_native.add_layer_norm, add_layer_norm_supported=_native.add_layer_norm_supported,
                           merge_weights=_native.merge_weights, merge_weights_supported=_native.merge_weights_supported,
                           channel_affine_gelu=_native.channel_affine_gelu,
                           channel_affine_gelu_supported=_native.channel_affine_gelu_supported,
                           add_row_score=_native.add_row_score, add_row_score_supported=_native.add_row_score_supported,
                           bias_table_grad=_native.bias_table_grad,
                           attn_softmax_backward=_native.attn_softmax_backward,
                           neighbour_lists=_native.neighbour_lists,
                           neighbour_lists_supported=_native.neighbour_lists_supported,
                           gather_rows=_native.gather_rows, gather_rows_supported=_native.gather_rows_supported,
                           merge_centres=_native.merge_centres, merge_centres_supported=_native.merge_centres_supported,
                           merge_rows=_native.merge_rows, merge_rows_supported=_native.merge_rows_supported)


def _cast_params(lin, dt):
    """(key, weight, bias) of an nn.Linear in dtype `dt`, kept until the parameters change."""
    key = (dt, lin.weight._version, lin.weight.data_ptr(),
           None if lin.bias is None else (lin.bias._version, lin.bias.data_ptr()))
    cache = lin.__dict__.get("_cast_cache")
    if cache is None or cache[0] != key:
        cache = (key, lin.weight.detach().to(dt), None if lin.bias is None else lin.bias.detach().to(dt))
        lin.__dict__["_cast_cache"] = cache      # a plain attribute: no parameter, no buffer, not in the state_dict
    return cache


def _linear(lin, x, ops=None, gelu=False):
    """`lin(x)` for an nn.Linear, followed by the exact GELU when `gelu`.  In inference under mixed precision the
    16-bit copies of weight and bias are kept between calls (autocast makes them anew in every forward; they are
    remade when the parameters change), and the small layers on many rows go through the library's kernel when
    `ops` has it."""
    if torch.is_grad_enabled() or not x.is_cuda or not torch.is_autocast_enabled("cuda"):
        y = lin(x)
        return F.gelu(y) if gelu else y
    dt = torch.get_autocast_dtype("cuda")
    cache = _cast_params(lin, dt)
    x = x if x.dtype == dt else x.to(dt)
    fn = getattr(ops, "linear", None)
    if fn is not None and ops.linear_supported(x, cache[1], gelu):
        return fn(x, cache[1], cache[2], gelu)
    y = F.linear(x, cache[1], cache[2])
    return F.gelu(y) if gelu else y


def _linear_pair(first, second, x, ops=None):
    """`(first(x), second(x))` for two nn.Linear layers that read the same input (the query and the key / value
    projections of an attention layer, aff_transformer.py:103-106).  In inference under mixed precision they run as
    one matrix product over the stacked 16-bit weights, kept between calls like the single copies; the results are
    the two column ranges of its output (views).  Layers that the library's small-layer kernel takes stay apart."""
    if (torch.is_grad_enabled() or not x.is_cuda or not torch.is_autocast_enabled("cuda")
            or first.bias is None or second.bias is None):
        return _linear(first, x, ops), _linear(second, x, ops)
    dt = torch.get_autocast_dtype("cuda")
    a, b = _cast_params(first, dt), _cast_params(second, dt)
    x = x if x.dtype == dt else x.to(dt)
    fn = getattr(ops, "linear", None)
    if fn is not None and ops.linear_supported(x, a[1], False) and ops.linear_supported(x, b[1], False):
        return fn(x, a[1], a[2], False), fn(x, b[1], b[2], False)
    key = (a[0], b[0])
    cache = first.__dict__.get("_pair_cache")
    if cache is None or cache[0] != key:
        cache = (key, torch.cat([a[1], b[1]], 0), torch.cat([a[2], b[2]], 0))
        first.__dict__["_pair_cache"] = cache    # a plain attribute, like _cast_cache
    y = F.linear(x, cache[1], cache[2])
    n_first = a[1].shape[0]
    return y[..., :n_first], y[..., n_first:]


def _layer_norm(norm, x, ops, feeds_linear=False):
    """`norm(x)` for an nn.LayerNorm; in inference on the GPU through the library's one-pass kernel when `ops` has it.

    `feeds_linear`: the result is only read by Linear layers, so under mixed precision it is produced in the
    autocast dtype directly (the rounding those layers would apply to their input, done once)."""
    fn = getattr(ops, "layer_norm", None)
    if fn is None or torch.is_grad_enabled() or not ops.layer_norm_supported(x):
        return norm(x)
    out_dtype = torch.get_autocast_dtype("cuda") if (feeds_linear and torch.is_autocast_enabled("cuda")) else None
    return fn(x, norm.weight, norm.bias, norm.eps, out_dtype)


def _one_pass_norm_available(ops, x):
    return (getattr(ops, "layer_norm", None) is not None and not torch.is_grad_enabled() and ops.layer_norm_supported(x))


def _add_layer_norm(norm, x, branch, ops):
    """(x + branch, norm(x + branch)) — just (x, norm(x)) when `branch` is None — with the norm's output feeding
    Linear layers only.  In inference under mixed precision addition and norm are one pass of the library's kernel
    when `ops` has it."""
    if branch is None:
        return x, _layer_norm(norm, x, ops, True)
    fn = getattr(ops, "add_layer_norm", None)
    if (fn is not None and not torch.is_grad_enabled() and torch.is_autocast_enabled("cuda")
            and branch.dtype == torch.get_autocast_dtype("cuda") and ops.add_layer_norm_supported(x, branch)):
        return fn(x, branch, norm.weight, norm.bias, norm.eps)
    x = x + branch
    return x, _layer_norm(norm, x, ops, True)


def _table_rows(table, idx):
    """table[idx] for a (rows, k) table and an index tensor of any shape, written as the reference writes it
    (aff_transformer.py:131: a `gather` along dim 0): the values are those of `table[idx]`, but the backward is a
    scatter-add, where the framework's backward of advanced indexing sorts the indices (19 ms per attention layer at
    batch 64 on this device: nine tenths of a training step)."""
    k = table.shape[1]
    return table.gather(0, idx.reshape(-1, 1).expand(-1, k)).reshape(*idx.shape, k)


class _PositionBias(torch.autograd.Function):
    """bias[pe_idx] laid out as (b, h, n, m), with the table's gradient from the library's kernel (sums per workgroup
    in LDS) instead of the framework's scatter-add of b*h*n*m values into a table of 12 000 rows."""

    @staticmethod
    def forward(ctx, bias, pe_idx, grad_kernel):
        ctx.save_for_backward(pe_idx)
        ctx.rows, ctx.dtype, ctx.grad_kernel = bias.shape[0], bias.dtype, grad_kernel
        return _table_rows(bias, pe_idx).permute(0, 3, 1, 2)

    @staticmethod
    def backward(ctx, grad):
        (pe_idx,) = ctx.saved_tensors
        return ctx.grad_kernel(grad, pe_idx, ctx.rows).to(ctx.dtype), None, None


class _AttnSoftmax(torch.autograd.Function):
    """Position bias, padding mask, blank token and softmax between QK and AV as one kernel forward and one backward
    (aff_transformer.py:125-147), with the bias table's gradient from `bias_table_grad`: the training counterpart of
    the inference path's `attn_softmax`."""

    @staticmethod
    def forward(ctx, attn, bias, pe_idx, mask, blank_logit, ops):
        probs, blank_prob = ops.attn_softmax(attn, bias, pe_idx, mask, blank_logit=blank_logit)
        ctx.save_for_backward(probs, blank_prob, pe_idx)
        ctx.meta = (attn.dtype, bias.shape[0], bias.dtype, blank_logit.dtype, ops)
        return probs, blank_prob

    @staticmethod
    def backward(ctx, d_probs, d_blank_prob):
        probs, blank_prob, pe_idx = ctx.saved_tensors
        attn_dtype, rows, bias_dtype, blank_dtype, ops = ctx.meta
        d_logit, d_blank = ops.attn_softmax_backward(probs, blank_prob, d_probs, d_blank_prob, attn_dtype)
        d_bias = ops.bias_table_grad(d_logit, pe_idx, rows).to(bias_dtype)
        return d_logit, d_bias, None, None, d_blank.to(blank_dtype), None


class _ClusterAttention(torch.autograd.Function):
    """The local attention of a block between its projections (aff_transformer.py:120-155) as one kernel forward and,
    backward, one kernel for the query side - the probabilities are recomputed from the softmax denominators the
    forward saved - followed by the sums that complete it: the scatters over the stage's sorted pair lists (d_key,
    d_value), the bias table's gradient, the blank token's.  No (b,h,n,m) tensor is kept between the two passes.
    The scatters go through the operators' own scatter, which reads the flag of the pair lists on the device: lists
    that turn out not to be made of whole clusters (never the model's own) take its atomic kernels, so d_key and d_value
    are complete sums whatever `member_idx` holds."""

    @staticmethod
    def forward(ctx, q, key, v, bias, blank_k, blank_v, plan, pairs, pe_idx, member_idx, scale, ops):
        out, lse = ops.cluster_attention(q, key, v, None, bias, None, None, blank_k, blank_v, scale=scale, plan=plan,
                                         return_lse=True)
        ctx.save_for_backward(q, key, v, out, lse, bias, blank_k, blank_v, plan, pairs, pe_idx, member_idx)
        ctx.meta = (scale, ops)
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, key, v, out, lse, bias, blank_k, blank_v, plan, pairs, pe_idx, member_idx = ctx.saved_tensors
        scale, ops = ctx.meta
        b, h, n, ch = q.shape
        d_q, probs, d_logit, blank_prob, d_blank = ops.cluster_attention_backward(
            q, key, v, d_out, out, lse, plan, bias, blank_k, blank_v, scale=scale)
        g = d_out.to(q.dtype).reshape(b, n, h, ch).permute(0, 2, 1, 3)
        d_v = ops.scatter_rows(probs, g, member_idx, pairs)
        d_k = ops.scatter_rows(d_logit, q, member_idx, pairs) * scale
        d_bias = ops.bias_table_grad(d_logit, pe_idx, bias.shape[0]).to(bias.dtype)
        d_bk = torch.einsum("bhn,bhnc->hc", d_blank, q.float()) * scale
        d_bv = torch.einsum("bhn,bhnc->hc", blank_prob, g.float())
        return (d_q, d_k.to(key.dtype), d_v.to(v.dtype), d_bias, d_bk.reshape(blank_k.shape).to(blank_k.dtype),
                d_bv.reshape(blank_v.shape).to(blank_v.dtype), None, None, None, None, None, None)


def _position_bias(bias, pe_idx, ops):
    """(b, h, n, m) position bias of an attention layer: row pe_idx[b,i,j] of the (rows, h) table for every pair."""
    kernel = getattr(ops, "bias_table_grad", None)
    if (kernel is not None and torch.is_grad_enabled() and bias.requires_grad and bias.is_cuda
            and bias.dtype in (torch.float32, torch.float16, torch.bfloat16)):
        return _PositionBias.apply(bias, pe_idx, kernel)
    return _table_rows(bias, pe_idx).permute(0, 3, 1, 2)


def _autocast_key():
    return torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else None


def _table_function(owner, slot, module, table, compute):
    """`compute()`, a function of `module`'s parameters and of the relative-position table only, kept between
    inference forwards: the position-bias table of an attention layer and the weight table of a merge are the same
    for every batch.  Recomputed when a parameter or the table changes (in place or by replacement) or the autocast
    state does; never kept while gradients are enabled."""
    if torch.is_grad_enabled() or not table.is_cuda:
        return compute()
    key = (tuple((q.data_ptr(), q._version) for q in module.parameters()), table.data_ptr(), table._version, table.dtype,
           _autocast_key())
    hit = owner.__dict__.get(slot)
    if hit is None or hit[0] != key:
        hit = (key, compute(), table)         # the table is held, so that its address cannot be reused by another one
        owner.__dict__[slot] = hit
    return hit[1]


def relative_position_table(img_size):
    """(table_width^2, 5) rows (dx, dy, distance, sin, cos) for every offset between two stride-4 tokens.

    aff_transformer.py:14-33: offsets range over [-R, R] with R = img_size // 4 - 1; the row of offset (dx, dy)
    is (dy + R) * (2R + 1) + (dx + R); the undefined angle at the origin is 0.
    """
    r = img_size // 4 - 1
    axis = torch.arange(2 * r + 1).float() - r
    dy, dx = torch.meshgrid(axis, axis, indexing="ij")
    dist = (dx ** 2 + dy ** 2) ** 0.5
    table = torch.stack([dx, dy, dist, dy / dist, dx / dist], dim=2)
    table[~torch.isfinite(table)] = 0
    return table.reshape(-1, 5), r


class DropPath(nn.Module):
    """Stochastic depth: drops the whole residual branch of a sample with probability p while training."""

    def __init__(self, p):
        super().__init__()
        self.p = float(p)

    def forward(self, x):
        if not self.training or self.p == 0.0:
            return x
        keep = 1.0 - self.p
        shape = (x.shape[0],) + (1,) * (x.dim() - 1)
        return x * x.new_empty(shape).bernoulli_(keep).div_(keep)


class Mlp(nn.Module):
    def __init__(self, dim, hidden, drop=0.0, ops=None):
        super().__init__()
        self.fc1 = nn.Linear(dim, hidden)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(hidden, dim)
        self.drop = nn.Dropout(drop)
        self.ops = ops

    def forward(self, x):
        hidden = _linear(self.fc1, x, self.ops, gelu=True)        # self.act is the exact GELU
        return self.drop(_linear(self.fc2, self.drop(hidden), self.ops))


class ClusterAttention(nn.Module):
    """Attention of every token over the members of its nearest clusters, plus one learned blank token."""

    def __init__(self, dim, num_heads, attn_drop=0.0, proj_drop=0.0, ops=None):
        super().__init__()
        self.dim, self.num_heads = dim, num_heads
        self.scale = (dim // num_heads) ** -0.5
        self.q = nn.Linear(dim, dim)
        self.kv = nn.Linear(dim, 2 * dim)
        self.blank_k = nn.Parameter(torch.randn(dim))
        self.blank_v = nn.Parameter(torch.randn(dim))
        self.pos_embed = nn.Linear(5, num_heads)
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(proj_drop)
        self.ops = ops
        self.cluster_size = 8     # tokens per cluster of the lists this layer is given (its stage sets it)

    def bias_table(self, table):
        """(rows, heads) position bias for every row of the relative-position table (aff_transformer.py:125-129)."""
        return _table_function(self, "_bias_table_cache", self.pos_embed, table, lambda: _linear(self.pos_embed, table))

    def forward(self, feat, member_idx, cluster_mask, pe_idx, global_attn, table, cluster_idx=None, grid_lists=None):
        """`grid_lists`: (cluster_idx, pe_idx, cluster_mask) with a leading 1 instead of the batch size, when the
        lists are the same for every image (tokens of a regular grid); the one-kernel path reads those."""
        b, n, c = feat.shape
        h = self.num_heads
        ch = c // h
        # inference: the neighbourhoods as (b,n,nnc) cluster numbers instead of the expanded (b,n,m*nnc) row lists
        numbered = cluster_idx is not None and not global_attn and not torch.is_grad_enabled()
        compact = numbered and getattr(self.ops, "qk_clusters", None) is not None
        sized = {} if self.cluster_size == 8 else {"cluster_size": self.cluster_size}
        q, kv = _linear_pair(self.q, self.kv, feat, self.ops)
        kv = kv.view(b, n, h, 2, ch).permute(3, 0, 2, 1, 4)                                                 # (2,b,h,n,ch) view
        key, v = kv[0], kv[1]
        one_kernel = getattr(self.ops, "cluster_attention", None)
        if (numbered and one_kernel is not None and not (self.training and self.attn_drop.p > 0)
                and self.ops.cluster_attention_supported(q.view(b, n, h, ch).permute(0, 2, 1, 3), cluster_idx.shape[2],
                                                         self.cluster_size)):
            # inference on 16-bit or fp32 data: scores, position bias, mask, blank token, softmax and the weighted sum
            # of the values in one kernel; the query scale is applied to the scores inside it
            lists = grid_lists if grid_lists is not None else (cluster_idx, pe_idx, cluster_mask)
            plan = lists[3] if len(lists) > 3 else None     # what the kernel makes of the lists, once per stage
            out = one_kernel(q.view(b, n, h, ch).permute(0, 2, 1, 3), key, v, lists[0], self.bias_table(table),
                             lists[1], lists[2], self.blank_k, self.blank_v, scale=self.scale,
                             **({"plan": plan} if plan is not None else {}))
            return self.proj_drop(_linear(self.proj, out, self.ops))
        train_kernel = getattr(self.ops, "cluster_attention_backward", None)
        if (train_kernel is not None and torch.is_grad_enabled() and cluster_idx is not None and not global_attn
                and self.cluster_size == 8 and grid_lists is not None and len(grid_lists) > 4 and not (self.training and self.attn_drop.p > 0)
                and self.ops.cluster_attention_backward_supported(q.view(b, n, h, ch).permute(0, 2, 1, 3),
                                                                  cluster_idx.shape[2])):
            # training: the same kernel forward, one kernel and four sums backward
            bias = self.bias_table(table)
            out = _ClusterAttention.apply(q.view(b, n, h, ch).permute(0, 2, 1, 3), key, v, bias, self.blank_k,
                                          self.blank_v, grid_lists[3], grid_lists[4], pe_idx, member_idx,
                                          self.scale, self.ops)
            return self.proj_drop(_linear(self.proj, out, self.ops))
        dense = getattr(self.ops, "dense_attention", None)
        if (global_attn and dense is not None and not torch.is_grad_enabled()
                and not (self.training and self.attn_drop.p > 0)
                and self.ops.dense_attention_supported(q.view(b, n, h, ch).permute(0, 2, 1, 3))):
            # inference on 16-bit data, every token attending to every token: one kernel as well
            out = dense(q.view(b, n, h, ch).permute(0, 2, 1, 3), key, v, self.bias_table(table), pe_idx,
                        self.blank_k, self.blank_v, scale=self.scale)
            return self.proj_drop(_linear(self.proj, out, self.ops))
        q = (q * self.scale).reshape(b, n, h, ch).permute(0, 2, 1, 3)                    # (b,h,n,ch) view
        if global_attn:
            attn = q @ key.transpose(-1, -2)                                             # (b,h,n,n)
        elif compact and self.ops.clusters_supported(q, cluster_idx.shape[2], **sized):
            attn = self.ops.qk_clusters(q, key, cluster_idx, **sized)                    # (b,h,n,m)
        else:
            compact = False
            attn = self.ops.qk(q, key, member_idx)                                       # (b,h,n,m)

        bias = self.bias_table(table)                                                     # (rows, h)
        fused = getattr(self.ops, "attn_softmax", None)
        if (fused is not None and not global_attn and not torch.is_grad_enabled()
                and not (self.training and self.attn_drop.p > 0) and self.ops.attn_softmax_supported(attn, attn.shape[-1])):
            # inference: bias gather, mask, blank-token logit and softmax in one kernel
            attn, blank = fused(attn, bias, pe_idx, cluster_mask, query=q, blank_key=self.blank_k)
        else:
            blank = (q * self.blank_k.reshape(1, h, 1, ch)).sum(-1, keepdim=True)        # (b,h,n,1)
            if (fused is not None and getattr(self.ops, "attn_softmax_backward", None) is not None
                    and getattr(self.ops, "bias_table_grad", None) is not None and torch.is_grad_enabled()
                    and not global_attn and attn.is_cuda
                    and not (self.training and self.attn_drop.p > 0)
                    and self.ops.attn_softmax_supported(attn, attn.shape[-1])):
                # training: the same glue as one kernel forward and one backward
                attn, blank = _AttnSoftmax.apply(attn, bias, pe_idx, cluster_mask, blank, self.ops)
            else:
                attn = attn + _position_bias(bias, pe_idx, self.ops)
                if cluster_mask is not None and not global_attn:
                    attn = attn + (1 - cluster_mask.reshape(b, 1, n, -1)) * (-100)
                attn = torch.softmax(torch.cat([attn, blank], dim=-1), dim=-1)
                attn = self.attn_drop(attn)
                blank, attn = attn[..., -1:], attn[..., :-1]

        if global_attn:
            out = attn @ v
        elif compact:
            out = self.ops.av_clusters(attn, v, cluster_idx, **sized)
        else:
            out = self.ops.av(attn, v, member_idx)                                       # (b,h,n,ch)
        out = out + blank * self.blank_v.reshape(1, h, 1, ch)
        out = out.permute(0, 2, 1, 3).reshape(b, n, c)
        return self.proj_drop(_linear(self.proj, out, self.ops))


class ClusterTransformerBlock(nn.Module):
    def __init__(self, dim, num_heads, mlp_ratio=2.0, drop=0.0, attn_drop=0.0, drop_path=0.0, layer_scale=0.0,
                 ops=None):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn = ClusterAttention(dim, num_heads, attn_drop=attn_drop, proj_drop=drop, ops=ops)
        self.drop_path = DropPath(drop_path) if drop_path > 0.0 else nn.Identity()
        self.norm2 = nn.LayerNorm(dim)
        self.mlp = Mlp(dim, int(dim * mlp_ratio), drop=drop, ops=ops)
        self.layer_scale = isinstance(layer_scale, (int, float)) and layer_scale > 0
        if self.layer_scale:
            self.gamma1 = nn.Parameter(layer_scale * torch.ones(dim))
            self.gamma2 = nn.Parameter(layer_scale * torch.ones(dim))

    def forward(self, feat, member_idx, cluster_mask, pe_idx, global_attn, table, cluster_idx=None, grid_lists=None,
                carry=None):
        """Returns (feat, branch): the block's output is feat + branch.  The addition is left to the caller, which
        hands `branch` to the next block as `carry` so that it can ride along with that block's first norm."""
        ops = self.attn.ops
        feat, x = _add_layer_norm(self.norm1, feat, carry, ops)
        a = self.attn(x, member_idx, cluster_mask, pe_idx, global_attn, table, cluster_idx, grid_lists)
        feat, x = _add_layer_norm(self.norm2, feat, self.drop_path(self.gamma1 * a if self.layer_scale else a), ops)
        f = self.mlp(x)
        return feat, self.drop_path(self.gamma2 * f if self.layer_scale else f)


class ClusterMerging(nn.Module):
    """Adaptive down-sampling: keeps ds_rate of the tokens and merges each one's neighbourhood into it."""

    INNER = 4

    def __init__(self, dim, out_dim, alpha=4.0, ds_rate=0.25, reserve_on=True, ops=None):
        super().__init__()
        self.alpha, self.ds_rate, self.reserve_on = alpha, ds_rate, reserve_on
        self.weight_net = nn.Sequential(nn.Linear(5, self.INNER), nn.LayerNorm(self.INNER), nn.GELU())
        self.norm = nn.LayerNorm(self.INNER * dim)
        self.linear = nn.Linear(self.INNER * dim, out_dim)
        self.ops = ops

    def select(self, pos, learned_prob, stride, reserve_num):
        """Indices (b, n') of the tokens kept as merge centres (aff_transformer.py:296-334)."""
        b, n, _ = pos.shape
        keep = int(n * self.ds_rate)
        one_pass = getattr(self.ops, "merge_centres", None)
        if one_pass is not None and self.ops.merge_centres_supported(pos, learned_prob):
            # scores, selection and the reserved tokens in one kernel; among equal scores at the cut the lower index
            dist = None if stride == 2 else knn(pos, pos, 2, return_dist=True)[1][:, :, 1]
            return one_pass(pos, dist, learned_prob, float(self.alpha), stride,
                            keep - reserve_num if self.reserve_on else keep, reserve_num, self.reserve_on)
        if stride == 2:                      # tokens still fill the grid: every other row and column
            prior = ((pos % stride).sum(-1) == 0).float()
        else:                                # adaptive grid: spacing from the distance to the nearest other token
            _, dist = knn(pos, pos, 2, return_dist=True)
            spacing = 2 ** (dist[:, :, 1].log2().ceil() + 1)
            prior = ((pos.long() % spacing.unsqueeze(2).long()).sum(-1) == 0).float()
        score = prior
        if learned_prob is not None:
            # widened before the addition (the values are those of the mixed-type addition; the framework's kernel
            # for mixed types has a fixed cost of some 45 us on this device, however small the tensors)
            score = score + (learned_prob.detach().view(b, n) * self.alpha).float()
        if not self.reserve_on:
            return score.topk(keep, dim=1, sorted=False)[1]
        reserved = ((pos % (stride * 2)).sum(-1) == 0)
        score = score + reserved.float() * (-100)
        sampled = score.topk(keep - reserve_num, dim=1, sorted=False)[1]
        # the reserved tokens in ascending index order; there are exactly reserve_num of them per image
        kept = reserved.to(torch.uint8).sort(dim=1, descending=True, stable=True)[1][:, :reserve_num]
        return torch.cat([sampled, kept], dim=1)

    def forward(self, pos, feat, member_idx, cluster_mask, learned_prob, stride, pe_idx, reserve_num, table):
        b, n, c = feat.shape
        m = member_idx.shape[-1]
        centre = self.select(pos, learned_prob, stride, reserve_num)                     # (b, n')
        n_out = centre.shape[1]
        assert n_out == int(n * self.ds_rate), "number of merge centres"
        rows_op = getattr(self.ops, "merge_rows", None)
        mask_rows = None
        if rows_op is not None and self.ops.merge_rows_supported(pos, member_idx, pe_idx):
            # the rows of the per-token tensors at the centres in one launch
            if cluster_mask is not None and self.ops.merge_rows_supported(cluster_mask):
                pos, member_idx, pe_idx, mask_rows = rows_op(centre, pos, member_idx, pe_idx, cluster_mask)
            else:
                pos, member_idx, pe_idx = rows_op(centre, pos, member_idx, pe_idx)
            rows = centre.unsqueeze(2).expand(-1, -1, m)
        else:
            pos = pos.gather(1, centre.unsqueeze(2).expand(-1, -1, pos.shape[2]))
            rows = centre.unsqueeze(2).expand(-1, -1, m)
            member_idx = member_idx.gather(1, rows)                                      # (b, n', m)
            pe_idx = pe_idx.gather(1, rows)
        if cluster_mask is not None and mask_rows is None:
            mask_rows = cluster_mask.gather(1, rows)
        table_w = _table_function(self, "_weight_table_cache", self.weight_net, table,
                                  lambda: self.weight_net(table))                         # (rows, 4)
        one_pass = getattr(self.ops, "merge_weights", None)
        if one_pass is not None and not torch.is_grad_enabled() and self.ops.merge_weights_supported(table_w):
            # inference: lookup, importance of each neighbour and mask in one kernel
            weights = one_pass(table_w, pe_idx, member_idx, learned_prob, mask_rows)
        else:
            weights = _table_rows(table_w, pe_idx)                                       # (b, n', m, 4)
            if learned_prob is not None:
                weights = weights * learned_prob.gather(1, member_idx.reshape(b, -1, 1)).reshape(b, n_out, m, 1)
            if cluster_mask is not None:
                weights = weights * mask_rows.unsqueeze(3)
        merged = self.ops.wf(weights, feat, member_idx).reshape(b, n_out, -1)            # channel = ic * c + c'
        return pos, _linear(self.linear, _layer_norm(self.norm, merged, self.ops, True), self.ops)


class BasicLayer(nn.Module):
    """One stage: neighbourhood lists, `depth` blocks over them, optional merging into the next stage."""

    def __init__(self, dim, out_dim, cluster_size, nbhd_size, depth, num_heads, mlp_ratio, alpha=4.0, ds_rate=0.25,
                 reserve_on=True, drop=0.0, attn_drop=0.0, drop_path=0.0, layer_scale=0.0, downsample=True,
                 ops=None):
        super().__init__()
        assert cluster_size > 0
        self.cluster_size, self.nbhd_size = cluster_size, nbhd_size
        self.ops = ops
        rates = drop_path if isinstance(drop_path, (list, tuple)) else [drop_path] * depth
        self.blocks = nn.ModuleList([
            ClusterTransformerBlock(dim, num_heads, mlp_ratio, drop, attn_drop, rates[i], layer_scale, ops=ops)
            for i in range(depth)])
        for blk in self.blocks:
            blk.attn.cluster_size = cluster_size
        if downsample:
            self.downsample = ClusterMerging(dim, out_dim, alpha, ds_rate, reserve_on, ops=ops)
            self.prob_net = nn.Linear(dim, 1)
        else:
            self.downsample = None
        self._grid_cache = {}

    def neighbourhoods(self, pos, h, w, radius, table_width):
        """(pos reordered, ranking or None, member_idx (b,n,nbhd), mask or None, pe_idx (b,n,nbhd),
        cluster numbers (b,n,nnc) int32 or None).

        aff_transformer.py:454-487.  The list of token i holds the members of its nnc nearest clusters,
        nearest cluster first; members of cluster g are tokens g*m .. g*m+m-1 of the reordered sequence.
        """
        b, n, d = pos.shape
        m = self.cluster_size
        k = int(math.ceil(n / float(m)))
        nnc = min(int(round(self.nbhd_size / float(m))), k)
        ranking = None
        if k == n:
            centres, members, mask = pos, torch.arange(n, device=pos.device).reshape(1, n, 1).expand(b, -1, -1), None
        else:
            pos, centres, members, mask, ranking = space_filling_cluster(pos, m, h, w)
        nearest = knn(pos, centres, nnc)                                                  # (b, n, nnc)
        one_pass = getattr(self.ops, "neighbour_lists", None)
        if (ranking is not None and one_pass is not None and not torch.is_grad_enabled()
                and self.ops.neighbour_lists_supported(pos, nearest)):
            # the four index tensors in one kernel
            member_idx, mask, pe_idx, cluster_idx = one_pass(pos, nearest, m, radius, table_width, mask is not None)
            return pos, ranking, member_idx, mask, pe_idx, (cluster_idx if m in (8, 24) else None)
        if ranking is not None:
            # cluster order: cluster g owns tokens g*m .. g*m+m-1, pad slots of the last one hold index 0 and mask 0
            rows = nearest.unsqueeze(3) * m + torch.arange(m, device=pos.device)
            valid = rows < n
            member_idx = torch.where(valid, rows, torch.zeros_like(rows)).reshape(b, n, nnc * m)
            if mask is not None:
                mask = valid.reshape(b, n, nnc * m).to(mask.dtype)
        else:
            pick = nearest.reshape(b, -1, 1).expand(-1, -1, m)
            member_idx = members.gather(1, pick).reshape(b, n, nnc * m)
            if mask is not None:
                mask = mask.gather(1, pick).reshape(b, n, nnc * m)
        nb_pos = pos.gather(1, member_idx.reshape(b, -1, 1).expand(-1, -1, d)).reshape(b, n, nnc * m, d)
        rel = nb_pos - (pos.unsqueeze(2) - radius)
        pe_idx = (rel[..., 1] * table_width + rel[..., 0]).long()
        # with clusters of m in cluster order, member_idx[b,i,m*r+t] = m*nearest[b,i,r]+t (0 past the last token):
        # the cluster numbers alone describe the lists (the kernels take clusters of 8 and, in part, of 24)
        cluster_idx = nearest.to(torch.int32).contiguous() if (ranking is not None and m in (8, 24)) else None
        return pos, ranking, member_idx, mask, pe_idx, cluster_idx

    def grid_order(self, pos1, h, w, radius):
        """The order (n,) in which this stage, as the first one, takes the tokens of the full grid (`pos1`: the
        positions of one image), or None when it leaves them as they are; fills the stage's cache of grid lists."""
        n = pos1.shape[1]
        if self.nbhd_size >= n:
            return None
        key = (n, h, w, str(pos1.device))
        if key not in self._grid_cache:
            self._grid_cache[key] = self.neighbourhoods(pos1[:1], h, w, radius, 2 * radius + 1)
        ranking = self._grid_cache[key][1]
        return None if ranking is None else ranking[0, :, 0]

    def forward(self, pos, feat, h, w, on_grid, stride, table, radius, feat_ordered=False):
        """`feat_ordered`: the tokens already stand in the order `grid_order` gave (first stage only)."""
        b, n, d = pos.shape
        table_width = 2 * radius + 1
        global_attn = self.nbhd_size >= n
        cluster_idx = grid_lists = None
        if global_attn:
            member_idx = mask = None
            rel = (pos[:, None, :, :] + radius) - pos[:, :, None, :]
            pe_idx = (rel[..., 1] * table_width + rel[..., 0]).long()
        else:
            if on_grid:
                # grid tokens are the same for every image: one image's lists serve the whole batch
                key = (n, h, w, str(pos.device))
                if key not in self._grid_cache:
                    self._grid_cache[key] = self.neighbourhoods(pos[:1], h, w, radius, table_width)
                pos1, ranking, member_idx, mask, pe_idx, cluster_idx = self._grid_cache[key]
                if (key, b) not in self._grid_cache:   # the batch-sized copies the operators read
                    self._grid_cache[(key, b)] = (member_idx.expand(b, -1, -1).contiguous(),
                                                  pe_idx.expand(b, -1, -1).contiguous(),
                                                  None if mask is None else mask.expand(b, -1, -1).contiguous(),
                                                  None if cluster_idx is None else cluster_idx.expand(b, -1, -1).contiguous())
                if cluster_idx is not None:
                    grid_lists = (cluster_idx, pe_idx, mask)           # one image's lists, for the one-kernel attention
                    planner = getattr(self.ops, "cluster_attention_plan", None)
                    if (planner is not None and not torch.is_grad_enabled() and cluster_idx.shape[2] == 6 and pe_idx.is_cuda
                            and (self.cluster_size == 8 or torch.is_autocast_enabled("cuda"))):
                        if (key, "plan") not in self._grid_cache:      # what that kernel makes of them, kept with them
                            self._grid_cache[(key, "plan")] = planner(cluster_idx, pe_idx, mask)
                        grid_lists = grid_lists + (self._grid_cache[(key, "plan")],)
                member_idx, pe_idx, mask, cluster_idx = self._grid_cache[(key, b)]
                pos = pos1.expand(b, -1, -1)
                if ranking is not None and not feat_ordered:
                    feat = feat[:, ranking[0, :, 0]]
            else:
                pos, ranking, member_idx, mask, pe_idx, cluster_idx = self.neighbourhoods(pos, h, w, radius, table_width)
                if ranking is not None:
                    rows_op = getattr(self.ops, "gather_rows", None)
                    if rows_op is not None and not torch.is_grad_enabled() and self.ops.gather_rows_supported(feat):
                        feat = rows_op(feat, ranking[:, :, 0])          # inference: one row-gather kernel
                    else:
                        feat = feat.gather(1, ranking.expand(-1, -1, feat.shape[2]))

        planner = getattr(self.ops, "cluster_attention_plan", None)
        if (grid_lists is None and cluster_idx is not None and planner is not None and not torch.is_grad_enabled()
                and cluster_idx.shape[2] == 6 and cluster_idx.is_cuda
                and ((feat.dtype == torch.float32 and self.cluster_size == 8) or torch.is_autocast_enabled("cuda"))):
            # the one-kernel attention of every block reads what it makes of the lists from a plan built once
            grid_lists = (cluster_idx, pe_idx, mask, planner(cluster_idx, pe_idx, mask))
        if ((grid_lists is None or len(grid_lists) == 3) and cluster_idx is not None and planner is not None
                and torch.is_grad_enabled() and getattr(self.ops, "cluster_attention_backward", None) is not None
                and not global_attn and self.cluster_size == 8 and cluster_idx.shape[2] == 6 and cluster_idx.is_cuda
                and (torch.is_autocast_enabled("cuda") or feat.dtype == torch.float32)):
            # training (fp32, or mixed precision): the plan of the one-kernel attention and the sorted pair lists of its
            # backward's scatters, built once for all blocks of the stage (a grid stage hands over one image's lists)
            pairs = self.ops.cluster_pairs(member_idx)
            if pairs is not None:
                lists = grid_lists if grid_lists is not None else (cluster_idx, pe_idx, mask)
                grid_lists = tuple(lists) + (planner(lists[0], lists[1], lists[2]), pairs)
        carry = None
        for blk in self.blocks:
            feat, carry = blk(feat, member_idx, mask, pe_idx, global_attn, table, cluster_idx, grid_lists, carry)
        learned_prob = None
        scorer = getattr(self.ops, "add_row_score", None)
        if (self.downsample is not None and scorer is not None and not torch.is_grad_enabled() and feat.is_cuda
                and torch.is_autocast_enabled("cuda")):
            # inference: the last residual addition and the importance score of the tokens in one pass
            _, w16, b16 = _cast_params(self.prob_net, torch.get_autocast_dtype("cuda"))
            if self.ops.add_row_score_supported(feat, carry, w16):
                feat, learned_prob = scorer(feat, carry, w16, b16)
                carry = None
        if carry is not None:
            feat = feat + carry

        if self.downsample is not None:
            if global_attn:   # merging after a dense stage: every token is every token's neighbour
                member_idx = torch.arange(n, device=feat.device).expand(b, n, n).contiguous()
            if learned_prob is None:
                learned_prob = _linear(self.prob_net, feat).sigmoid()
            reserve_num = math.ceil(h / (stride * 2)) * math.ceil(w / (stride * 2))
            pos, feat = self.downsample(pos, feat, member_idx, mask, learned_prob, stride, pe_idx, reserve_num, table)
        return pos, feat


class PatchEmbed(nn.Module):
    """Two stride-2 3x3 convolutions (BatchNorm + GELU between them): one token per 4x4 pixels."""

    def __init__(self, in_chans=3, embed_dim=32, patch_norm=True, ops=None):
        super().__init__()
        self.ops = ops
        self.proj1 = nn.Conv2d(in_chans, embed_dim // 2, kernel_size=3, stride=2, padding=1)
        self.bn = nn.BatchNorm2d(embed_dim // 2)
        self.act1 = nn.GELU()
        self.proj2 = nn.Conv2d(embed_dim // 2, embed_dim, kernel_size=3, stride=2, padding=1)
        self.norm = nn.LayerNorm(embed_dim) if patch_norm else None

    def _bn_affine(self):
        """BatchNorm in inference as y = x * scale + shift per channel, the first convolution's bias folded in; kept
        until a parameter or a running statistic changes."""
        bn, conv = self.bn, self.proj1
        parts = [t for t in (bn.weight, bn.bias, bn.running_mean, bn.running_var, conv.bias) if t is not None]
        key = tuple((t.data_ptr(), t._version) for t in parts)
        hit = self.__dict__.get("_bn_affine_cache")
        if hit is None or hit[0] != key:
            scale = torch.rsqrt(bn.running_var.float() + bn.eps)
            if bn.weight is not None:
                scale = scale * bn.weight.float()
            shift = -bn.running_mean.float() if conv.bias is None else conv.bias.float() - bn.running_mean.float()
            shift = shift * scale
            if bn.bias is not None:
                shift = shift + bn.bias.float()
            hit = (key, scale.detach(), shift.detach())
            self.__dict__["_bn_affine_cache"] = hit
        return hit[1], hit[2]

    def forward(self, x, token_order=None):
        """`token_order(pos_of_one_image, h, w)`, when given, returns the order (N,) in which the first stage wants
        the tokens (or None); the tokens then leave in that order when the final norm can take it along, and the
        fifth return value says whether they did."""
        fused = getattr(self.ops, "channel_affine_gelu", None)
        if (fused is not None and not torch.is_grad_enabled() and not self.bn.training and x.is_cuda
                and torch.is_autocast_enabled("cuda") and self.bn.track_running_stats):
            # inference: bias, BatchNorm (an affine map per channel) and GELU in one pass over the convolution's output
            y = F.conv2d(x, self.proj1.weight, None, self.proj1.stride, self.proj1.padding)
            if self.ops.channel_affine_gelu_supported(y):
                y = fused(y, *self._bn_affine())
            else:
                y = self.act1(self.bn(y if self.proj1.bias is None else y + self.proj1.bias.view(1, -1, 1, 1)))
        else:
            y = self.act1(self.bn(self.proj1(x)))
        b, _, h0, w0 = y.shape
        h, w = (h0 + 1) // 2, (w0 + 1) // 2
        ys, xs = torch.meshgrid(torch.arange(h, device=x.device), torch.arange(w, device=x.device), indexing="ij")
        pos = torch.stack([xs, ys], dim=2).reshape(1, -1, 2)
        order = None
        if self.norm is not None and token_order is not None and x.is_cuda and not torch.is_grad_enabled():
            order = token_order(pos.float(), h, w)
        if order is not None or (self.norm is not None and self.proj2.bias is not None and x.is_cuda
                                 and not torch.is_grad_enabled()):
            # the second convolution's bias and the reordering ride along with the norm
            z = F.conv2d(y, self.proj2.weight, None, self.proj2.stride, self.proj2.padding)
            z = z.flatten(2).transpose(1, 2).contiguous()
            if _one_pass_norm_available(self.ops, z):
                tokens = self.ops.layer_norm(z, self.norm.weight, self.norm.bias, self.norm.eps, None, order,
                                             self.proj2.bias)
                return pos.expand(b, -1, -1).to(tokens.dtype), tokens, h, w, order is not None
            if self.proj2.bias is not None:
                z = z + self.proj2.bias
            tokens = self.norm(z)
            return pos.expand(b, -1, -1).to(tokens.dtype), tokens, h, w, False
        tokens = self.proj2(y).flatten(2).transpose(1, 2)
        assert tokens.shape[1] == h * w
        if self.norm is not None:
            tokens = _layer_norm(self.norm, tokens, self.ops)
        return pos.expand(b, -1, -1).to(tokens.dtype), tokens, h, w, False


class AutoFocusFormer(nn.Module):
    """aff_transformer.py:560-670.  Defaults are the reference's; `aff_tiny()` gives configs/aff_tiny.yaml."""

    def __init__(self, in_chans=3, num_classes=1000, embed_dim=(32, 128, 256, 512), cluster_size=8,
                 nbhd_size=(48, 48, 48, 49), alpha=4.0, ds_rate=0.25, reserve_on=True, depths=(2, 2, 6, 2),
                 num_heads=(3, 6, 12, 24), mlp_ratio=2.0, drop_rate=0.0, attn_drop_rate=0.0, drop_path_rate=0.1,
                 patch_norm=True, layer_scale=0.0, img_size=224, ops=None):
        super().__init__()
        ops = ops if ops is not None else default_ops()
        self.num_classes = num_classes
        self.num_features = embed_dim[-1]
        self.ops = ops
        self.patch_embed = PatchEmbed(in_chans, embed_dim[0], patch_norm, ops=ops)
        self.pos_drop = nn.Dropout(drop_rate)
        table, self.radius = relative_position_table(img_size)
        self.register_buffer("pre_table", table, persistent=False)
        rates = [r.item() for r in torch.linspace(0, drop_path_rate, sum(depths))]
        last = len(depths) - 1
        self.layers = nn.ModuleList([
            BasicLayer(embed_dim[i], embed_dim[i + 1] if i < last else None, cluster_size, nbhd_size[i], depths[i],
                       num_heads[i], mlp_ratio, alpha, ds_rate, reserve_on, drop_rate, attn_drop_rate,
                       rates[sum(depths[:i]):sum(depths[:i + 1])], layer_scale, downsample=i < last, ops=ops)
            for i in range(len(depths))])
        self.norm = nn.LayerNorm(self.num_features)
        self.head = nn.Linear(self.num_features, num_classes) if num_classes > 0 else nn.Identity()
        self.apply(self._init_weights)

    @staticmethod
    def _init_weights(mod):
        if isinstance(mod, nn.Linear):
            nn.init.trunc_normal_(mod.weight, std=0.02)
            if mod.bias is not None:
                nn.init.zeros_(mod.bias)
        elif isinstance(mod, nn.LayerNorm):
            nn.init.zeros_(mod.bias)
            nn.init.ones_(mod.weight)

    def forward_features(self, x):
        first = self.layers[0]
        pos, x, h, w, ordered = self.patch_embed(x, lambda pos1, h, w: first.grid_order(pos1, h, w, self.radius))
        x = self.pos_drop(x)
        table = self.pre_table
        if not torch.is_grad_enabled() and table.is_cuda and torch.is_autocast_enabled("cuda"):
            # every block's position-embedding Linear would round the table to 16 bits again: one copy, kept
            dt = torch.get_autocast_dtype("cuda")
            key = (table.data_ptr(), table._version, dt)
            hit = self.__dict__.get("_table_cast_cache")
            if hit is None or hit[0] != key:
                hit = (key, table.to(dt))
                self.__dict__["_table_cast_cache"] = hit
            table = hit[1]
        for i, layer in enumerate(self.layers):
            pos, x = layer(pos, x, h, w, on_grid=(i == 0), stride=2 ** (i + 1), table=table, radius=self.radius,
                           feat_ordered=(i == 0 and ordered))
        return _layer_norm(self.norm, x, self.ops).mean(1)

    def forward(self, x):
        x = self.forward_features(x)
        return _linear(self.head, x) if isinstance(self.head, nn.Linear) else x


def aff_tiny(**kw):
    """configs/aff_tiny.yaml: depths 3/4/18/5, dims 64/128/256/512, heads 2/4/8/16, mlp ratio 3, 48 neighbours."""
    cfg = dict(embed_dim=(64, 128, 256, 512), depths=(3, 4, 18, 5), num_heads=(2, 4, 8, 16), mlp_ratio=3.0,
               cluster_size=8, nbhd_size=(48, 48, 48, 49), alpha=4.0, ds_rate=0.25, drop_path_rate=0.2)
    cfg.update(kw)
    return AutoFocusFormer(**cfg)


class CapturedForward:
    """One inference forward of `net` at a fixed input shape, recorded into a HIP graph and replayed.

    A forward of the classifier is some 800 kernel launches of 5-100 us each; issued one by one from Python they
    take as long on the host as on the GPU.  Replaying the recorded graph leaves one launch per forward.  The
    model's forward has no host synchronisation and every kernel of the library takes the current stream and
    allocates through the framework, so the recording is the plain forward under `torch.cuda.graph`.

    Replays read the parameters in place (their 16-bit copies are part of the recording: record again after the
    weights change) and return the same output tensor every time: copy it before the next call if it must outlive
    it.  `autocast_dtype=None` records without mixed precision.
    """

    def __init__(self, net, example, autocast_dtype=torch.float16, warmup=3):
        if not example.is_cuda:
            raise RuntimeError("CapturedForward records GPU work: the example input must be a CUDA tensor")
        self.net = net
        self.autocast_dtype = autocast_dtype
        self.static_in = example.clone()
        side = torch.cuda.Stream(device=example.device)
        side.wait_stream(torch.cuda.current_stream(example.device))
        with torch.cuda.stream(side):        # library handles, kernel selection and caches settle outside the recording
            for _ in range(warmup):
                self._forward()
        torch.cuda.current_stream(example.device).wait_stream(side)
        torch.cuda.synchronize(example.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_out = self._forward()

    def _forward(self):
        with torch.no_grad(), torch.autocast("cuda", dtype=self.autocast_dtype or torch.float16,
                                            enabled=self.autocast_dtype is not None):
            return self.net(self.static_in)

    def __call__(self, x):
        if x.shape != self.static_in.shape or x.dtype != self.static_in.dtype:
            raise RuntimeError("CapturedForward was recorded for inputs of shape %s and dtype %s"
                               % (tuple(self.static_in.shape), self.static_in.dtype))
        if x.data_ptr() != self.static_in.data_ptr():
            self.static_in.copy_(x)
        self.graph.replay()
        return self.static_out
