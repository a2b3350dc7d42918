"""Synthetic gradient sets (shapes only) and the fusion planner used to form
fusion cycles for tests and benchmarks.

The planner restates Controller::FuseResponses of the reference
(common/controller.cc:793-866) for one dtype and one set of scale factors:
tensors join the open group in arrival order while the 16-byte padded total
stays within the threshold; a tensor that does not fit ends the group unless
the look-ahead budget still covers it, in which case later tensors may still
join.  A tensor larger than the threshold is a single-entry response, which
the ops run tensor -> output with no fusion buffer (ops/nccl_operations.cc:176-186).
"""
import math

import numpy as np

FUSION_THRESHOLD = 64 * 1024 * 1024


def resnet50_shapes():
    """torchvision ResNet-50 parameters in named_parameters() order:
    161 tensors, 25,557,032 elements."""
    shapes = [(64, 3, 7, 7), (64,), (64,)]
    inplanes = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            shapes += [(planes, inplanes, 1, 1), (planes,), (planes,),
                       (planes, planes, 3, 3), (planes,), (planes,),
                       (planes * 4, planes, 1, 1), (planes * 4,), (planes * 4,)]
            if b == 0:
                shapes += [(planes * 4, inplanes, 1, 1), (planes * 4,), (planes * 4,)]
            inplanes = planes * 4
    shapes += [(1000, 2048), (1000,)]
    return shapes


def bert_large_shapes():
    """BERT-large-shaped set of 397 tensors (the nominal "340M" elements):
    5 embedding tensors, 24 layers x 16 tensors, pooler (2), masked-LM head
    (transform dense w/b, LayerNorm w/b, decoder bias; the decoder weight is
    tied to the word embedding) and the next-sentence classifier weight."""
    h, ff = 1024, 4096
    shapes = [(30522, h), (512, h), (2, h), (h,), (h,)]
    for _ in range(24):
        shapes += [(h, h), (h,), (h, h), (h,), (h, h), (h,), (h, h), (h,), (h,), (h,),
                   (ff, h), (ff,), (h, ff), (h,), (h,), (h,)]
    shapes += [(h, h), (h,)]                      # pooler
    shapes += [(h, h), (h,), (h,), (h,), (30522,)]  # MLM transform dense + LayerNorm + decoder bias
    shapes += [(2, h)]                            # next-sentence classifier weight
    assert len(shapes) == 397
    return shapes


def gpt2_xl_shapes():
    """GPT-2 XL: 580 tensors, 1,557,611,200 elements."""
    d = 1600
    shapes = [(50257, d), (1024, d)]
    for _ in range(48):
        shapes += [(d,), (d,), (d, 3 * d), (3 * d,), (d, d), (d,), (d,), (d,), (d, 4 * d), (4 * d,), (4 * d, d), (d,)]
    shapes += [(d,), (d,)]
    assert len(shapes) == 580
    return shapes


def stress_counts(seed=3, n=1024, lo=256, hi=65536):
    """Element counts log-uniform in [lo, hi]."""
    rng = np.random.default_rng(seed)
    return [int(round(math.exp(u))) for u in rng.uniform(math.log(lo), math.log(hi), n)]


def adasum_layer_counts(total=1 << 25, nlayers=64, seed=13):
    """A seeded random composition of `total` into nlayers parts, each >= 1."""
    rng = np.random.default_rng(seed)
    cuts = np.sort(rng.choice(np.arange(1, total), nlayers - 1, replace=False))
    bounds = np.concatenate([[0], cuts, [total]])
    counts = [int(x) for x in np.diff(bounds)]
    assert sum(counts) == total and min(counts) >= 1
    return counts


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


FUSION_BUFFER_ATOMIC_UNIT = 64  # common/common.h:146


def reduce_scatter_share(num_elements, world, fused=True):
    """Elements of one GPU's share of the reduce-scatter over a buffer of num_elements, as
    NCCLHierarchicalAllreduce::Execute cuts it (ops/nccl_operations.cc:285-316).  A fused response
    first grows to a multiple of world * 64 elements (the extra ones are dummy elements behind the
    payload, inside the fusion buffer, whose size the planner keeps divisible); every rank then owns
    num_elements / world consecutive elements starting at rank * share.  A single tensor is not
    grown: its remainder num_elements % world goes through a separate reduce at the last rank."""
    if fused:
        div = world * FUSION_BUFFER_ATOMIC_UNIT
        num_elements = (num_elements + div - 1) // div * div
    return num_elements // world


def reduce_scatter_ranges(num_elements, world, fused=True):
    """(first element, count) of what every local rank reduces, in rank order, as
    NCCLHierarchicalAllreduce::Execute cuts a homogeneous job (ops/nccl_operations.cc:285-330): rank r
    owns the share at r * share (buffer_data_at_rank_offset); the elements that do not divide
    (single tensors only, a fused buffer is grown first) sit behind the last share and are reduced at
    the last rank (root_rank = local_size - 1), whose range therefore runs to the end of the buffer."""
    share = reduce_scatter_share(num_elements, world, fused)
    if fused:
        return [(r * share, share) for r in range(world)]
    rest = num_elements % world
    return [(r * share, share + (rest if r == world - 1 else 0)) for r in range(world)]


def fuse(nbytes, threshold=FUSION_THRESHOLD, pad16=True):
    """Greedy fusion of a list of tensor byte sizes (one dtype, one set of scale
    factors) into groups of tensor indices, in the reference's queue discipline."""
    pad = (lambda s: 16 * ((s + 15) // 16)) if pad16 else (lambda s: s)
    group_of = [-1] * len(nbytes)
    groups = []
    for head in range(len(nbytes)):
        if group_of[head] != -1:
            continue
        g = len(groups)
        groups.append([head])
        group_of[head] = g
        size = pad(nbytes[head])
        skipped = 0
        for j in range(head + 1, len(nbytes)):
            if group_of[j] != -1:
                continue
            nsz = pad(nbytes[j])
            if size + nsz <= threshold:
                size += nsz
                group_of[j] = g
                groups[g].append(j)
            else:
                skipped += nsz
                if size + skipped > threshold:
                    break
    return groups
