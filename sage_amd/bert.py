"""BERT: host-side mirror of models/bert.rs.

`reference_exact=True` (default) composes exactly what the reference composes, including what
differs from a textbook BERT: ReLU in the feed-forward block (bert.rs:192), LayerNorm with scalar
gamma = beta and eps 1e-05 (layers.rs:563-590), no segment embedding (bert.rs:97-102), the
classifier reads token index 1 (bert.rs:76), no pooler.  `reference_exact=False` builds the
configuration the benchmark names from the same operators: erf-GELU, per-feature LayerNorm with
the configured eps, an optional segment table, classifier on token 0.
"""
import numpy as np

from .layers import Dense, Dropout, Embedding, Gelu, Layer, LayerNorm, Relu, Sequential, Softmax
from .tensor import FLOAT, UINT, Tensor
from .var import Var, into_var


class BertConfig:
    """bert.rs:8-54."""

    def __init__(self, embed_dim, num_vocabs, max_num_tokens, hidden_dim, num_layers, num_attention_heads,
                 layer_norm_eps, dropout_prob, num_classes):
        self.embed_dim, self.num_vocabs, self.max_num_tokens = embed_dim, num_vocabs, max_num_tokens
        self.hidden_dim, self.num_layers, self.num_attention_heads = hidden_dim, num_layers, num_attention_heads
        self.layer_norm_eps, self.dropout_prob, self.num_classes = layer_norm_eps, dropout_prob, num_classes

    @staticmethod
    def simple():
        return BertConfig(64, 150, 512, 128, 6, 2, 0.0, 0.0, 10)

    @staticmethod
    def base():
        return BertConfig(768, 30522, 512, 3072, 12, 12, 1e-12, 0.3, 2)


class MultiHeadAttention(Layer):
    """bert.rs:206-314."""

    def __init__(self, embed_dim, num_heads, dropout_prob, layer_norm_eps, reference_exact=True):
        self.embed_dim, self.num_heads, self.head_dim = embed_dim, num_heads, embed_dim // num_heads
        self.key_proj = Dense(embed_dim, embed_dim)
        self.query_proj = Dense(embed_dim, embed_dim)
        self.value_proj = Dense(embed_dim, embed_dim)
        self.attn_softmax = Softmax(3)
        self.dense = Dense(embed_dim, embed_dim)
        self.dropout = Dropout(dropout_prob)
        self.norm = LayerNorm(2, layer_norm_eps, embed_dim, reference_exact)

    def params(self):
        return (self.key_proj.params() + self.query_proj.params() + self.value_proj.params()
                + self.dense.params() + self.norm.params())

    def separate_heads(self, f):
        """bert.rs:282-291: (N,L,H*D) -> (N,L,H,D) -> (N,H,L,D), zero-copy."""
        n, l = f.extent(0), f.extent(1)
        return f.view([n, l, self.num_heads, self.head_dim]).transpose(2, 1)

    def merge_heads(self, f):
        """bert.rs:293-302."""
        f = f.transpose(2, 1)
        n, l = f.extent(0), f.extent(1)
        return f.view([n, l, self.num_heads * self.head_dim])

    def extend_mask(self, mask):
        """bert.rs:304-314: (N,L) -> (N,1,1,L); (1 - mask) * -1e5."""
        n, l = mask.extent(0), mask.extent(1)
        m = mask.view([n, 1, 1, l])
        return (-m + 1.0) * -1e5

    def pass_(self, x, attn_mask):
        q = self.separate_heads(self.query_proj.pass_(x))
        k = self.separate_heads(self.key_proj.pass_(x))
        v = self.separate_heads(self.value_proj.pass_(x))
        att = q.matmul_batched(k.transpose(-1, -2)) / float(np.sqrt(np.float32(self.head_dim)))
        att = self.attn_softmax.pass_(att + self.extend_mask(attn_mask))
        av = self.merge_heads(att.matmul_batched(v))
        y = self.dense.pass_(av)
        return self.norm.pass_(y + x)


class BertLayer(Layer):
    """bert.rs:175-204."""

    def __init__(self, config, reference_exact=True):
        self.attention = MultiHeadAttention(config.embed_dim, config.num_attention_heads, config.dropout_prob,
                                            config.layer_norm_eps, reference_exact)
        self.ffn = Sequential(Dense(config.embed_dim, config.hidden_dim),
                              Relu() if reference_exact else Gelu(),
                              Dense(config.hidden_dim, config.embed_dim),
                              Dropout(config.dropout_prob))
        self.norm = LayerNorm(2, config.layer_norm_eps, config.embed_dim, reference_exact)

    def params(self):
        return self.attention.params() + self.ffn.params() + self.norm.params()

    def pass_(self, x, attn_mask):
        interim = self.attention.pass_(x, attn_mask)
        out = self.ffn.pass_(interim)
        return self.norm.pass_(out + interim)


class BertEmbedding(Layer):
    """bert.rs:83-140."""

    def __init__(self, config, reference_exact=True, segments=0):
        self.word_emb = Embedding(config.num_vocabs, config.embed_dim)
        self.pos_emb = Embedding(config.max_num_tokens, config.embed_dim)
        self.seg_emb = Embedding(segments, config.embed_dim) if segments else None
        self.norm = LayerNorm(2, config.layer_norm_eps, config.embed_dim, reference_exact)

    def params(self):
        p = self.word_emb.params() + self.pos_emb.params()
        if self.seg_emb is not None:
            p += self.seg_emb.params()
        return p + self.norm.params()

    def pass_(self, ids, ctx, segment_ids=None):
        ids = into_var(ids)
        l = ids.extent(1)
        pos = Var.new(Tensor.from_numpy(ctx, np.arange(l, dtype=np.uint32)))  # bert.rs:131
        e = self.word_emb.pass_(ids) + self.pos_emb.pass_(pos)
        if self.seg_emb is not None and segment_ids is not None:
            e = e + self.seg_emb.pass_(segment_ids)
        return self.norm.pass_(e)


class Bert(Layer):
    """bert.rs:56-81."""

    def __init__(self, config, reference_exact=True, segments=0):
        self.config = config
        self.reference_exact = reference_exact
        self.embedding = BertEmbedding(config, reference_exact, segments)
        self.layers = [BertLayer(config, reference_exact) for _ in range(config.num_layers)]
        self.classifier = Dense(config.embed_dim, config.num_classes)

    def params(self):
        p = self.embedding.params()
        for l in self.layers:
            p += l.params()
        return p + self.classifier.params()

    def encode(self, x, attn_mask):
        for l in self.layers:
            x = l.pass_(x, attn_mask)
        return x

    def classify(self, f):
        """bert.rs:76-79: the classifier reads one token of the last encoder output."""
        cls = f.index(1, 1 if self.reference_exact else 0).squeeze(1)
        return self.classifier.pass_(cls)

    def pass_(self, token_ids, attn_mask, ctx, segment_ids=None):
        e = self.embedding.pass_(token_ids, ctx, segment_ids)
        return self.classify(self.encode(e, into_var(attn_mask)))
