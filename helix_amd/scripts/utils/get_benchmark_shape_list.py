"""Workload shape tables for the op-level and model-level benchmarks.

Same four entry points and return structure as the reference's
scripts/utils/get_benchmark_shape_list.py (:1, :17, :29, :38), so the benchmark wrappers iterate them
the same way.  GEMM shapes are (M, N, K); conv shapes are
(batch, IC, H, W, OC, kH, kW, stride, pad).  The lists are composed in the reference's order from a few
generators (token counts x projection sizes, graph tables x hidden sizes, batch lists x per-layer
tables); the long per-layer and DeepBench tables are plain data in benchmark_shapes.json next to this
file.  The five benchmark configurations this backend is measured on are the BASELINE_* names below.
"""
import json
import os

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "benchmark_shapes.json")) as _f:
    _TABLES = json.load(_f)


def _tuples(name):
    return [tuple(row) for row in _TABLES[name]]


# decode / prefill token counts the reference sweeps: 60 values, mostly primes, from 2 to 1949
TOKEN_COUNTS = [2, 13, 31, 53, 73, 101, 127, 151, 179, 199, 233, 263, 283, 317, 353, 383, 419, 443, 467, 503, 547,
                577, 607, 641, 661, 701, 739, 769, 811, 839, 877, 911, 947, 983, 1019, 1049, 1087, 1109, 1153, 1193,
                1229, 1277, 1297, 1321, 1381, 1429, 1453, 1487, 1521, 1559, 1597, 1621, 1663, 1697, 1739, 1783,
                1823, 1871, 1902, 1949]

# (N, K) of transformer projections: BERT-large, BERT-base, GPT-3-13B-like, LLaMA-2-7B
TRANSFORMER_NK = [(1024, 1024), (4096, 1024), (1024, 4096), (768, 2304), (3072, 768), (768, 3072), (768, 768),
                  (4096, 4096), (15360, 5120), (5120, 5120), (13824, 5120), (5120, 13824), (12288, 4096),
                  (4096, 4096), (11008, 4096), (4096, 11008)]

CNN_FC_BATCHES = [1, 2, 4, 8, 16, 32, 64, 128]
CNN_FC_NK = [(12544, 120), (120, 80), (80, 10), (9216, 4096), (4096, 4096), (4096, 1000), (25088, 4096),
             (512, 1000), (1024, 1000), (25088, 1000)]

CNN_BATCHES = [1, 4, 8, 12, 16, 20, 24, 28, 32, 36, 40, 44, 48, 52, 56, 60, 64]

ALEXNET_LAYERS = [(3, 224, 224, 96, 11, 11, 4, 0), (96, 26, 26, 256, 5, 5, 1, 2), (256, 12, 12, 384, 3, 3, 1, 1),
                  (384, 12, 12, 384, 3, 3, 1, 1), (384, 12, 12, 256, 3, 3, 1, 1)]
GOOGLENET_LAYERS = _tuples("googlenet_layers")
VGG_LAYERS = _tuples("vgg_layers")
RESNET_LAYERS = _tuples("resnet_layers")
DEEPBENCH_CONV = _tuples("deepbench_conv")
DEEPBENCH_GEMM = _tuples("deepbench_gemm")
GNN_GRAPHS = _tuples("gnn_graphs")          # (nodes, input features, classes)
GNN_HIDDEN = list(_TABLES["gnn_hidden"])

# ---- the five measured configurations ------------------------------------------------------------
BASELINE_SQUARE_SIZES = [1024, 2048, 4096, 8192]
BASELINE_GEMV_BATCHES = [1, 4, 16]
BASELINE_GEMV_KN = [(4096, 4096), (4096, 11008), (11008, 4096), (8192, 28672)]       # weight K x N
BASELINE_RESNET50_LAYERS = [(64, 56, 56, 64, 3, 3, 1, 1), (64, 56, 56, 256, 1, 1, 1, 0),
                            (128, 28, 28, 128, 3, 3, 1, 1), (256, 14, 14, 256, 3, 3, 1, 1),
                            (512, 7, 7, 512, 3, 3, 1, 1), (256, 56, 56, 512, 1, 1, 2, 0)]
BASELINE_CONV_BATCH = 32
BASELINE_BERT_M = 4096                                                                # batch 8 x seq 512
BASELINE_BERT_LAYER_NK = [(2304, 768), (768, 768), (3072, 768), (768, 3072)]          # QKV, out, FFN1, FFN2
BASELINE_BERT_LAYERS = 12
BASELINE_IRREGULAR_MNK = (4000, 2300, 770)


def gnn_MNKList():
    """Two-layer GCN feature transforms: per hidden size, X[nodes x features] * W1 for every graph, then
    H[nodes x hidden] * W2 for every graph."""
    out = []
    for hidden in GNN_HIDDEN:
        out += [(nodes, hidden, features) for (nodes, features, _) in GNN_GRAPHS]
        out += [(nodes, classes, hidden) for (nodes, _, classes) in GNN_GRAPHS]
    return out


def get_gemm_op_MNKList():
    transformer = [(m, n, k) for m in TOKEN_COUNTS for (n, k) in TRANSFORMER_NK]
    cnn_fc = [(m, n, k) for m in CNN_FC_BATCHES for (n, k) in CNN_FC_NK]
    return transformer + cnn_fc + DEEPBENCH_GEMM + gnn_MNKList()


def get_llm_opset_MNKList():
    bert_nk = [(768, 768)] * 49 + [(768, 3072)] * 12 + [(3072, 768)] * 12
    llama2_nk = [(12288, 4096), (4096, 4096), (11008, 4096), (4096, 11008)]
    gpt2_nk = [(768, 2304)] * 24 + [(3072, 768)] * 48 + [(768, 3072)] * 24
    bert = [(m, n, k) for m in TOKEN_COUNTS for (n, k) in bert_nk]
    llama2 = [(m, n, k) for m in TOKEN_COUNTS for (n, k) in llama2_nk]
    gpt2 = [(m, n, k) for m in TOKEN_COUNTS for (n, k) in gpt2_nk]
    return bert, llama2, gpt2


def get_conv_op_shape_list():
    layers = ALEXNET_LAYERS + GOOGLENET_LAYERS + VGG_LAYERS + RESNET_LAYERS
    return [(batch,) + shape for batch in CNN_BATCHES for shape in layers] + DEEPBENCH_CONV


def get_cnn_opset_shape_List():
    """(AlexNet, ResNet, GoogleNet) per-layer lists over the batch sweep."""
    alexnet = [(batch,) + shape for batch in CNN_BATCHES for shape in ALEXNET_LAYERS]
    resnet = [(batch,) + shape for batch in CNN_BATCHES for shape in RESNET_LAYERS]
    googlenet = [(batch,) + shape for batch in CNN_BATCHES for shape in GOOGLENET_LAYERS]
    return alexnet, resnet, googlenet


def get_baseline_bert_MNKList():
    """config 5: BERT-base encoder GEMMs at batch 8, seq 512, x12 layers, plus the irregular shape."""
    per_layer = [(BASELINE_BERT_M, n, k) for (n, k) in BASELINE_BERT_LAYER_NK]
    return per_layer * BASELINE_BERT_LAYERS + [BASELINE_IRREGULAR_MNK]


def get_baseline_conv_shape_list():
    """config 4: batch-32 NHWC ResNet-50-shaped layers."""
    return [(BASELINE_CONV_BATCH,) + shape for shape in BASELINE_RESNET50_LAYERS]
