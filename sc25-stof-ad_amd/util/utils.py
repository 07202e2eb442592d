"""The live helpers of the reference's ``src/util/utils.py`` (:8-47) under the same names."""
import timeit

import torch


def torch_cuda_identify(print_info=True):
    """src/util/utils.py:8-17."""
    if torch.cuda.is_available():
        if print_info:
            print(' PyTorch version:', torch.__version__)
            print(' HIP version \t:', torch.version.hip)
            print(' GPU cuda:({}) \t: {}'.format(torch.cuda.current_device(), torch.cuda.get_device_name()),
                  '\n', "-" * 50)
        return torch.device('cuda:{}'.format(torch.cuda.current_device()))
    print('cuda is not avaliable !')
    return torch.device('cpu')


def time_stamp_cudasync():
    """src/util/utils.py:19-21."""
    torch.cuda.synchronize()
    return timeit.default_timer()


def set_dtype(ts, dtype):
    """src/util/utils.py:23-28."""
    if dtype == "fp32":
        return ts.float()
    if dtype == "fp16":
        return ts.half()
    raise RuntimeError(f"Unsupported dtype {dtype}")


def transpose_for_scores(x, n_heads, head_size):
    """src/util/utils.py:30-34: (B,S,H*W) -> (B,H,S,W) view."""
    return x.view(x.size()[:-1] + (n_heads, head_size)).permute(0, 2, 1, 3)


def seqlen_to_mask(lengths, max_len):
    """src/util/utils.py:41-47: [B] lengths -> [B,max_len] bool, True where position < length."""
    batch_size = lengths.numel()
    return (torch.arange(0, max_len, device=lengths.device).type_as(lengths)
            .repeat(batch_size, 1).lt(lengths.unsqueeze(1)))
