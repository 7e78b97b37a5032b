"""``Cuda_BERT``: the encoder object the serving engine holds, one per GPU.

Same constructor, ``encode`` and teardown behaviour as the reference class
(cuda_model.py:4-41); ``config`` needs the attributes ``is_large``,
``model_npy_pth``, ``batch_size`` and ``max_seq_length`` (config.py:6-39).
"""
import numpy as np

from . import pybert


class Cuda_BERT(object):
    def __init__(self, id_gpu, config):
        self.id_gpu = id_gpu
        self.max_batchsize = config.batch_size
        self.max_seq_length = config.max_seq_length
        self.hidden_size = 1024 if config.is_large else 768
        self.model = pybert.load_model(config.is_large, config.model_npy_pth, id_gpu,
                                       config.batch_size, config.max_seq_length)
        self.cu_encode = pybert.bert

    def encode(self, input_tensor):
        """input_tensor: (input_ids, segment_ids, mask), each numpy int32
        [batchsize, seq_length].  Returns the pooled output [batchsize, hidden]."""
        indexed_tokens = np.ascontiguousarray(input_tensor[0], dtype=np.int32)
        segments_ids = np.ascontiguousarray(input_tensor[1], dtype=np.int32)
        attention_mask = np.ascontiguousarray(input_tensor[2], dtype=np.int32)
        batchsize, seq_length = indexed_tokens.shape
        output = np.ones([batchsize, self.hidden_size]).astype(np.float32)
        self.cu_encode(self.model, output, indexed_tokens, segments_ids,
                       batchsize, seq_length, attention_mask)
        return output

    def __del__(self):
        model = getattr(self, "model", None)
        if model:
            pybert.unload_model(model)
            self.model = None
