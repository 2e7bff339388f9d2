"""Variable-length batch metadata shared by every operator (mirrors upstream flash_nsa/utils.py:139-282).

NSAHelper is process-global state, as upstream: module constructors set the hyper-parameters, a forward call
registers the batch's cu_seqlens, and the operators read the derived compressed-row / selection-block offsets.
"""
import torch


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def cu_seqlens_to_seqlens(cu):
    return cu[1:] - cu[:-1]


def seqlens_to_cu_seqlens(seqlens):
    out = torch.zeros(seqlens.numel() + 1, dtype=torch.int32, device=seqlens.device)
    out[1:] = torch.cumsum(seqlens, 0)
    return out


class NSAHelper:
    kernel_size = 32
    stride = 16
    block_size = 64
    window_size = 512
    top_n = 16
    num_init_blocks = 1
    num_local_blocks = 2

    recompute_swa_o = False
    recompute_slc_o = False
    recompute_cmp_kv = False
    recompute_cmp_o = False

    cmp_k_method = "mean"
    cmp_v_method = "mean"

    pp_size = 1
    world_size = 1
    rank = 0
    process_group = None
    bench_mode = False

    x_cu_seqlens = None
    x_seqlens = None
    x_maxlen = 0
    y_cu_seqlens = None
    y_seqlens = None
    y_maxlen = 0
    y_len = 0
    k_cu_seqlens = None
    k_seqlens = None
    k_maxlen = 0
    k_len = 0
    blk_seq = None  # [k_len] sequence id of every selection block (used by the inverse index)
    batch = 0
    deterministic = False       # dk / dv summed in a fixed order instead of with atomics (set_deterministic)
    _registered = None          # the cu_seqlens tensor object of the registered batch and its version counter
    _registered_version = -1
    _host_cu = None

    @classmethod
    def set_hyperparameters(cls, kernel_size=32, stride=16, block_size=64, window_size=512, top_n=16,
                            num_init_blocks=1, num_local_blocks=2):
        changed = (cls.kernel_size, cls.stride, cls.block_size) != (kernel_size, stride, block_size)
        cls.kernel_size = kernel_size
        cls.stride = stride
        cls.block_size = block_size
        cls.window_size = window_size
        cls.top_n = top_n
        cls.num_init_blocks = num_init_blocks
        cls.num_local_blocks = num_local_blocks
        if changed:
            cls._registered = None
            cls.x_cu_seqlens = None

    @classmethod
    def set_recompute(cls, recompute_swa_o=False, recompute_slc_o=False, recompute_cmp_kv=False,
                      recompute_cmp_o=False):
        cls.recompute_swa_o = recompute_swa_o
        cls.recompute_slc_o = recompute_slc_o
        cls.recompute_cmp_kv = recompute_cmp_kv
        cls.recompute_cmp_o = recompute_cmp_o

    @classmethod
    def set_deterministic(cls, deterministic=True):
        """dK / dV of the compressed and the selected branch summed in a run-independent order (what upstream's
        dkdv_repeat=True buys): the backward kernels store per-work-item partial results that a second launch adds in
        a fixed order, instead of fp32 atomic additions.  Costs scratch memory and a few per cent of the backward."""
        cls.deterministic = bool(deterministic)

    @classmethod
    def set_pipeline_parallel_world_size(cls, pp_size):
        cls.pp_size = pp_size

    @classmethod
    def set_context_parallel(cls, process_group=None, kv_head_stride=1, use_overlap_swa=True):
        if process_group is not None:
            raise NotImplementedError("context parallelism is outside this single-GPU build")

    @classmethod
    def set_cmp_kv_method(cls, cmp_k_method, cmp_v_method):
        cls.cmp_k_method = cmp_k_method
        cls.cmp_v_method = cmp_v_method

    @classmethod
    def enable_bench_mode(cls):
        cls.bench_mode = True

    @classmethod
    def disable_bench_mode(cls):
        cls.bench_mode = False

    @classmethod
    def _need_init(cls, cu):
        """False when `cu` holds the registered lengths (upstream flash_nsa/utils.py:216-226 compares values).
        The same, unmodified tensor object is recognised without a device read; the helper keeps a reference to it,
        so its address cannot be handed to another tensor in the meantime."""
        if cls.x_cu_seqlens is None:
            return True
        if cu is cls._registered and cu._version == cls._registered_version:
            return False
        if cu.numel() != len(cls._host_cu):
            return True
        return [int(v) for v in cu.tolist()] != cls._host_cu

    @classmethod
    def init_cu_seqlens(cls, x_cu_seqlens: torch.Tensor, x_cu_seqlens_np=None, cp_mode=1):
        """Registers a packed batch: cu_seqlens int tensor [B+1] with cu[0]=0, cu[-1]=T."""
        if not cls._need_init(x_cu_seqlens):
            cls._registered, cls._registered_version = x_cu_seqlens, x_cu_seqlens._version
            return
        host = [int(v) for v in x_cu_seqlens.tolist()]
        assert len(host) >= 2 and host[0] == 0, "cu_seqlens must start at 0"
        dev = x_cu_seqlens.device
        xs = [host[i + 1] - host[i] for i in range(len(host) - 1)]
        assert all(l >= 0 for l in xs), "cu_seqlens must be non-decreasing"
        ys = [max((l - cls.kernel_size) // cls.stride + 1, 0) for l in xs]
        ks = [cdiv(l, cls.block_size) for l in xs]

        def cum(v):
            out = [0]
            for e in v:
                out.append(out[-1] + e)
            return out

        cls.batch = len(xs)
        cls.x_cu_seqlens = x_cu_seqlens.to(torch.int32).contiguous()
        cls.x_seqlens = torch.tensor(xs, dtype=torch.int32, device=dev)
        cls.x_maxlen = max(xs)
        cls.y_seqlens = torch.tensor(ys, dtype=torch.int32, device=dev)
        cls.y_cu_seqlens = torch.tensor(cum(ys), dtype=torch.int32, device=dev)
        cls.y_maxlen = max(ys)
        cls.y_len = sum(ys)
        cls.k_seqlens = torch.tensor(ks, dtype=torch.int32, device=dev)
        cls.k_cu_seqlens = torch.tensor(cum(ks), dtype=torch.int32, device=dev)
        cls.k_maxlen = max(ks)
        cls.k_len = sum(ks)
        cls.blk_seq = torch.repeat_interleave(torch.arange(len(ks), dtype=torch.int32), torch.tensor(ks)).to(
            device=dev, dtype=torch.int32)
        cls._host_cu = host
        cls._registered, cls._registered_version = x_cu_seqlens, x_cu_seqlens._version

    @classmethod
    def clear_tensor_data(cls, *tensors):
        for t in tensors:
            if isinstance(t, torch.Tensor):
                t.data = torch.empty(0, dtype=t.dtype, device=t.device)

    @classmethod
    def get_bwd_helper(cls):
        return cls if cls.pp_size <= 1 else BwdNSAHelper()


class BwdNSAHelper:
    """Snapshot of the batch metadata taken at forward time, for schedules that interleave micro-batches
    between a forward and its backward (upstream flash_nsa/utils.py:465-482)."""
    _FIELDS = ("kernel_size", "stride", "block_size", "window_size", "top_n", "num_init_blocks", "num_local_blocks",
               "x_cu_seqlens", "x_seqlens", "x_maxlen", "y_cu_seqlens", "y_seqlens", "y_maxlen", "y_len",
               "k_cu_seqlens", "k_seqlens", "k_maxlen", "k_len", "blk_seq", "batch", "cmp_k_method", "cmp_v_method",
               "deterministic")

    def __init__(self):
        for f in self._FIELDS:
            setattr(self, f, getattr(NSAHelper, f))
