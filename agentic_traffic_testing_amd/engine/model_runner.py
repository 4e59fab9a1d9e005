"""Model runner: KV-cache allocation, per-step input preparation, hipGraph decode replay.

One step = one forward over a decode-first ``Batch`` (scheduler.py) followed by sampling.

* **KV cache** - one [L, nb, Hkv, BS, D] K tensor and one [L, nb, Hkv, D, BS] V tensor (V
  transposed for the PV MFMA, see ops/csrc/attention.hip).  ``num_blocks`` comes from
  ``gpu_memory_utilization`` of the device's HBM after weights and an activation reserve,
  i.e. ~1.9 M tokens for Llama-3-8B at 0.9 of 288 GB.
* **Metadata** - the native block manager emits int32 arrays which are packed into ONE
  pinned host buffer and moved with ONE async H2D copy per step; every device metadata
  tensor is a view into the matching device buffer.
* **hipGraphs** - decode-only steps are padded to a bucket (1, 2, 4, 8, ...) and replayed
  from a captured graph that contains the whole forward, the LM head and the sampler, so a
  decode step costs one graph launch instead of ~330 kernel launches.
* **Tensor parallelism** - rank 0 owns scheduler + block manager; every step it packs the
  same int32 metadata it uploads into a step message (header + payload) and publishes it
  on a shared-memory channel (runtime/csrc/shm_channel.cpp).  TP worker ranks
  (``serve_worker``) replay exactly the same kernel / collective sequence from it, graph
  captures included, so the RCCL all-reduces line up.
"""
from __future__ import annotations

import math
import os
import threading
import time

import numpy as np
import torch

from .. import ops
from ..config import EngineConfig, ModelConfig
from ..models import model_class
from ..models.llama import AttnMeta, torch_dtype
from .state_cache import HybridCache
from ..ops import reference as ref
from ..runtime import BlockManager
from .scheduler import Batch


def _even(n: int) -> int:
    return n + (n & 1)


class MetaLayout:
    """int32-word layout of the packed per-step metadata buffer."""

    def __init__(self, T: int, S: int, W: int, NT: int):
        self.T, self.S, self.W, self.NT = T, S, W, NT
        o = 0
        self.fields = {}

        def add(name, n, dtype=torch.int32):
            nonlocal o
            words = n * (2 if dtype == torch.int64 else 1)
            if dtype == torch.int64:
                o = _even(o)
            self.fields[name] = (o, n, dtype)
            o += words

        add("input_ids", T)
        add("positions", T)
        add("slot_mapping", T)
        add("block_tables", S * W)
        add("seq_kvlen", S)
        add("seq_qstart", S + 1)
        add("seq_slot", S)
        add("tile_seq", NT)
        add("tile_qoff", NT)
        add("feed_prev", 1)     # 1: decode rows take the previous step's device samples
        add("temperature", S, torch.float32)
        add("top_p", S, torch.float32)  # >= 1: off
        add("top_k", S)                 # <= 0: off
        add("logits_idx", S, torch.int64)
        add("seeds", S, torch.int64)
        add("steps", S, torch.int64)
        self.size = _even(o)

    def views(self, buf: torch.Tensor) -> dict:
        out = {}
        for name, (o, n, dt) in self.fields.items():
            if dt == torch.int64:
                out[name] = buf[o:o + 2 * n].view(torch.int64)
            elif dt == torch.float32:
                out[name] = buf[o:o + n].view(torch.float32)
            else:
                out[name] = buf[o:o + n]
        out["block_tables"] = out["block_tables"].view(self.S, self.W)
        return out

    def pack(self, host: np.ndarray, arrays: dict):
        for name, (o, n, dt) in self.fields.items():
            a = arrays.get(name)
            if a is None:
                continue
            if dt == torch.int64:
                host[o:o + 2 * n].view(np.int64)[:len(a)] = a
            elif dt == torch.float32:
                host[o:o + n].view(np.float32)[:len(a)] = a
            else:
                host[o:o + n][:a.size] = a.reshape(-1)


# step-message header (int32 words) shared by rank 0 and the TP workers
HDR_WORDS = 12
OP_STEP, OP_CAPTURE, OP_STOP, OP_BARRIER = 1, 2, 3, 4


class ModelRunner:
    def __init__(self, cfg: EngineConfig, model_cfg: ModelConfig, device: str = "cuda",
                 comm=None, weights_dir=None):
        self.cfg = cfg
        self.mcfg = model_cfg
        self.device = torch.device(device)
        self.is_cuda = self.device.type == "cuda"
        self.dtype = torch_dtype(cfg.dtype)
        self.comm = comm
        tp_rank, tp_size = (comm.rank, comm.size) if comm is not None else (0, 1)
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.publisher = None     # rank 0 of a TP group: ShmChannel to the workers
        t0 = time.perf_counter()
        self.model = model_class(model_cfg.family)(model_cfg, self.dtype, self.device, tp_rank,
                                                    tp_size, comm, quantization=cfg.quantization)
        # hybrid models keep per-sequence state (recurrent layers, convolution tails) in state
        # slots next to the paged KV pool; their step runs the mixer op layer
        self.hybrid = bool(getattr(self.model, "has_state", False))
        self.cache: HybridCache | None = None
        self.model.prefill_gemm = cfg.prefill_gemm
        self.model.prefill_gemm_min_rows = cfg.prefill_gemm_min_rows
        self.model.small_prefill_fused = cfg.small_prefill_fused
        # tuned library-GEMM table (agentic_traffic_testing_amd/tuning): prefill steps pad
        # their rows to its buckets so their GEMMs hit tuned shapes
        self.gemm_table = None
        if self.device.type == "cuda" and cfg.gemm_tuning and not self.hybrid:
            from .. import tuning

            self.gemm_table = tuning.load(cfg.gemm_tuning, model_cfg.name)
        self.model.gemm_tuned = self.gemm_table is not None
        if weights_dir and cfg.load_format != "dummy":
            self.model.load_safetensors(weights_dir)
        else:
            self.model.init_random(seed=cfg.seed)
        if self.is_cuda and not self.hybrid and (
                (cfg.fused_decode and cfg.preshuffle_decode_weights
                 and self._room_for_decode_copies()) or cfg.quantization == "fp8"):
            self.model.prepare_decode_weights()
        self.load_seconds = time.perf_counter() - t0
        if self.is_cuda and not self.hybrid:
            # split-K GEMV workspace up front (32 MiB): a split chosen while a decode graph is
            # being captured (ATTA_DECODE_KSPLIT, TP shards) must not allocate inside the capture
            ops.ensure_splitk_workspace(self.device)
            if cfg.fused_decode:
                ops.warm_wide_kernels(self.device, self.dtype)
            if cfg.startup_warmup:
                self.warm_library_gemms()
        self.block_size = cfg.block_size
        self.bt_width = math.ceil(cfg.max_model_len / cfg.block_size)
        self.part_tokens = cfg.decode_partition_tokens
        self.max_parts = max(1, math.ceil(cfg.max_model_len / self.part_tokens))
        # small decode batches split the context finer (more workgroups in flight for the
        # latency-bound attention): partition tiers by batch size, finest first - the optional
        # tiny tier (<= decode_tiny_batch_max, 64 tokens; off by default, see config.py) and
        # small (<= decode_small_batch_max, 128 tokens); partial buffers are sized for the
        # finest split
        self.part_tiers = []  # (max batch, partition tokens, max partitions, graph buckets)
        for mb, pt in ((cfg.decode_tiny_batch_max, cfg.decode_partition_tokens_tiny),
                       (cfg.decode_small_batch_max, cfg.decode_partition_tokens_small)):
            if mb <= 0 or not pt or pt == self.part_tokens:
                continue
            mp = max(1, math.ceil(cfg.max_model_len / pt))
            if mp > 64:  # in-kernel combine handles <= 64 partitions
                continue
            bk = sorted({p for p in cfg.graph_parts_buckets if p < mp} | {mp})
            self.part_tiers.append((mb, pt, mp, bk))
        alloc_parts = max([self.max_parts] + [t[2] for t in self.part_tiers])
        # decode graphs are captured per (batch bucket, partition bucket): the attention grid
        # is (seqs, kv heads, partitions) and every workgroup past a sequence's context still
        # costs a dispatch and a round trip - a 32-partition grid (max_model_len 8192) over
        # 3k-token contexts ran 2.6x the workgroups it needed
        # (profiles/r2_fused_qkv_attn_experiment.txt: B=8 attention 21.9 us vs 10.8 at B=1)
        self.parts_buckets = sorted({p for p in cfg.graph_parts_buckets if p < self.max_parts}
                                    | {self.max_parts})
        self.tile_tokens = (self.model.attn_tile_tokens if self.hybrid else
                            ops.prefill_tile_tokens(self.model.g, bt_width=self.bt_width))
        self.graph_sizes = sorted(b for b in cfg.graph_batch_sizes)
        cap = next((b for b in self.graph_sizes if b >= cfg.max_num_seqs), cfg.max_num_seqs)
        self.graph_sizes = [b for b in self.graph_sizes if b <= cap]
        self.max_seqs = max(cfg.max_num_seqs, self.graph_sizes[-1] if self.graph_sizes else 1)
        self.max_tokens = cfg.max_num_batched_tokens + self.max_seqs
        if self.is_cuda and cfg.gemm_tuning and not self.hybrid:  # room for prefill row padding
            from ..tuning import bucket_rows

            self.max_tokens = bucket_rows(self.max_tokens)
        if self.hybrid:
            # decode attention partitions are the mixer kernels' (one size for every batch)
            from ..ops import mixers as _mx

            self.part_tokens = _mx.DECODE_PART_TOKENS
            self.max_parts = max(1, math.ceil(cfg.max_model_len / self.part_tokens))
            self.part_tiers = []
            self.parts_buckets = sorted({p for p in cfg.graph_parts_buckets if p < self.max_parts}
                                        | {self.max_parts})
            # a cached prefix would skip tokens whose recurrent state was never computed
            self._alloc_hybrid()
            self.bm = BlockManager(self.num_blocks, self.block_size, False, self.max_seqs)
        else:
            self._alloc_kv()
            self.bm = BlockManager(self.num_blocks, self.block_size, cfg.enable_prefix_caching)
        # metadata buffers (max layout)
        self.max_layout = MetaLayout(self.max_tokens, self.max_seqs, self.bt_width,
                                     self.max_tokens)
        pin = self.is_cuda
        # two pinned metadata buffers, used alternately: a step's H2D copy may still be queued
        # while the host packs the next step (async look-ahead decode, TP workers); an event
        # per buffer orders reuse behind the copy that last read it
        self.meta_hosts = [torch.zeros(self.max_layout.size, dtype=torch.int32, pin_memory=pin)
                           for _ in range(2)]
        self.meta_hosts_np = [h.numpy() for h in self.meta_hosts]
        self._mh = 0
        self._h2d_done = [torch.cuda.Event() if self.is_cuda else None for _ in range(2)]
        self.meta_dev = torch.zeros(self.max_layout.size, dtype=torch.int32, device=self.device)
        # sampled tokens of in-flight steps land here (D2H, one slot per in-flight step)
        self.tok_host = [torch.zeros(max(cfg.max_num_seqs, 256), dtype=torch.int64,
                                     pin_memory=pin) for _ in range(2)]
        self._tok_done = [torch.cuda.Event() if self.is_cuda else None for _ in range(2)]
        # the prefill GEMM's error word as of the last prefill step (0: every wait succeeded)
        self._err_host = torch.zeros(1, dtype=torch.int32, pin_memory=pin)
        # OR of the words read since the last take_kernel_error() (the device word is cleared
        # on every read), and how many steps ever reported one
        self.kernel_error = 0
        self.kernel_error_steps = 0
        # the engine thread ORs words in, the HTTP loop's /health swaps them out
        self._kernel_error_lock = threading.Lock()
        self._last_collect = 0.0
        self.graphs: dict[tuple, torch.cuda.CUDAGraph] = {}
        self.graph_io: dict[tuple, dict] = {}
        self.graph_pool = None
        self.steps = 0
        self.graph_steps = 0
        self.timing = {"graph_prep": 0.0, "graph_run": 0.0}
        self.fused_decode = False
        if self.hybrid:
            # sampled tokens of a step land here, as for every other model
            self.ws = {"tokens": torch.zeros(self.max_seqs, dtype=torch.int64,
                                             device=self.device)}
            return
        nkv = self.model.n_kv_heads
        self.part_out = torch.empty(self.max_seqs * nkv * alloc_parts * 16 * 128,
                                    dtype=torch.float32, device=self.device)
        self.part_lse = torch.empty(self.max_seqs * nkv * alloc_parts * 16,
                                    dtype=torch.float32, device=self.device)
        # fused decode-path workspace (q / attention / activation rows, sampler keys,
        # split-K partials and arrival counters for the decode attention kernel)
        H = self.mcfg.hidden_size
        dt, dev = self.dtype, self.device
        self.ws = {
            "q": torch.empty(self.max_seqs, self.model.n_heads, 128, dtype=dt, device=dev),
            "attn": torch.empty(self.max_seqs, self.model.n_heads, 128, dtype=dt, device=dev),
            "act": torch.empty(self.max_seqs, self.model.inter, dtype=dt, device=dev),
            "keys": torch.zeros(self.max_seqs * (self.model.vocab_shard // 16 + 1),
                                dtype=torch.int64, device=dev),
            "tokens": torch.zeros(self.max_seqs, dtype=torch.int64, device=dev),
            "tp_keys": torch.zeros(self.max_seqs, dtype=torch.int64, device=dev),
            "counters": torch.zeros(self.max_seqs * nkv, dtype=torch.int32, device=dev),
            "part_out": self.part_out, "part_lse": self.part_lse,
            "max_parts": self.max_parts, "part_tokens": self.part_tokens,
        }
        del H
        # the fused decode attention combines <= 64 partitions in-kernel (<= 16k tokens at
        # 256-token partitions); longer contexts use the two-kernel split-K path
        self.fused_decode = bool(cfg.fused_decode) and self.max_parts <= 64
        self.model.fused_decode = self.fused_decode
        # graphs are keyed (batch bucket, partition bucket, sampler variant)

    def _room_for_decode_copies(self) -> bool:
        """The pre-shuffled decode copies double the 16-bit weights (16 GB for Llama-3.1-8B);
        Llama-3-70B bf16 on ONE GPU (141 GB) cannot afford a second copy next to its KV cache,
        so it decodes from the row-major weights instead."""
        need = self.model.decode_copy_bytes()
        torch.cuda.synchronize(self.device)
        free, total = torch.cuda.mem_get_info(self.device)
        keep = max(int(0.15 * total), 24 << 30)  # KV cache + activations + graphs
        ok = int(need <= free - keep)
        if self.comm is not None and self.comm.size > 1:
            # every TP rank must pick the same GEMV layout (ranks sharing a GPU, or loading at
            # different times, see different free memory): the group decides by MIN
            ok = self.comm.min_int(ok, self.device)
        if not ok:
            print(f"[atta] skipping pre-shuffled decode weights: {need / 2**30:.1f} GiB needed, "
                  f"{free / 2**30:.1f} GiB free (row-major decode GEMVs)", flush=True)
            return False
        return True

    # ------------------------------------------------------------------------------------
    def _alloc_kv(self):
        m = self.model
        L = self.mcfg.num_layers
        per_block = 2 * L * m.n_kv_heads * self.block_size * m.head_dim * self.dtype.itemsize
        if self.cfg.num_kv_blocks > 0:
            nb = self.cfg.num_kv_blocks
        elif self.is_cuda:
            torch.cuda.synchronize()
            free, total = torch.cuda.mem_get_info(self.device)
            used = total - free
            # activation / workspace reserve: logits + GEMM intermediates at the token budget
            T = self.cfg.max_num_batched_tokens
            act = T * (self.mcfg.hidden_size * 8 + (m.inter * 2 + m.qkv_width) * 2) * 2
            act += self.max_seqs_estimate() * self.mcfg.vocab_size * 4 * 2 + (2 << 30)
            budget = total * self.cfg.gpu_memory_utilization - used - act
            if self.cfg.tp_same_device and self.tp_size > 1:
                # every rank shares this one device (the one-GPU TP rehearsal): each gets its
                # share of the budget, charged for its own allocations only (the ranks probe
                # free memory at different moments)
                mine = torch.cuda.memory_reserved(self.device)
                budget = total * self.cfg.gpu_memory_utilization / self.tp_size - mine - act
            nb = int(budget // per_block)
        else:
            nb = int(os.environ.get("ATTA_CPU_KV_BLOCKS", "256"))
        nb = max(nb, 2 * self.bt_width)
        if self.comm is not None:  # TP ranks must agree on the page count
            nb = self.comm.min_int(nb, self.device)
        self.num_blocks = nb
        shape_k = (L, nb, m.n_kv_heads, self.block_size, m.head_dim)
        shape_v = (L, nb, m.n_kv_heads, m.head_dim, self.block_size)
        # zero-init (tidy, not required: the attention kernels zero the V of every key past a
        # sequence's end before P.V, so stale or non-finite bytes there are harmless)
        self.k_cache = torch.zeros(shape_k, dtype=self.dtype, device=self.device)
        self.v_cache = torch.zeros(shape_v, dtype=self.dtype, device=self.device)
        self.k_layers = [self.k_cache[i] for i in range(L)]
        self.v_layers = [self.v_cache[i] for i in range(L)]
        self.kv_bytes = per_block * nb

    def _alloc_hybrid(self):
        """Page pool and state slots of a hybrid model: the pool takes what
        ``gpu_memory_utilization`` leaves after the weights, an activation reserve and the
        state slots (one per admissible sequence)."""
        specs = self.model.cache_specs()
        item = self.dtype.itemsize
        per_block = sum(sp.page_bytes(self.block_size, item) for sp in specs)
        slots = self.max_seqs
        slot_bytes = sum(sp.slot_bytes(item) for sp in specs) * slots
        if self.cfg.num_kv_blocks > 0:
            nb = self.cfg.num_kv_blocks
        elif self.is_cuda and per_block > 0:
            torch.cuda.synchronize()
            free, total = torch.cuda.mem_get_info(self.device)
            T = self.cfg.max_num_batched_tokens
            act = T * self.mcfg.hidden_size * 64 + self.max_seqs_estimate() * \
                self.mcfg.vocab_size * 8 + (2 << 30)
            budget = total * self.cfg.gpu_memory_utilization - (total - free) - act - slot_bytes
            nb = int(budget // per_block)
        else:
            nb = int(os.environ.get("ATTA_CPU_KV_BLOCKS", "256"))
        nb = max(nb, 2 * self.bt_width if self.cfg.num_kv_blocks <= 0 else 1)
        self.num_blocks = nb
        self.cache = HybridCache.allocate(specs, nb, self.block_size, slots, self.dtype,
                                          self.device)
        self.kv_bytes = self.cache.nbytes()

    def max_seqs_estimate(self) -> int:
        return max(self.cfg.max_num_seqs, 16)

    @property
    def kv_total_tokens(self) -> int:
        return self.num_blocks * self.block_size

    # ------------------------------------------------------------------------------------
    def _tier(self, batch_size: int) -> tuple:
        """(partition tokens, max partitions, graph partition buckets) of a decode step of
        ``batch_size`` rows (the graph bucket when replayed)."""
        for mb, pt, mp, bk in self.part_tiers:
            if 0 < batch_size <= mb:
                return pt, mp, bk
        return self.part_tokens, self.max_parts, self.parts_buckets

    def _ws_for(self, batch_size: int) -> dict:
        pt, mp, _ = self._tier(batch_size)
        if pt == self.part_tokens:
            return self.ws
        return {**self.ws, "part_tokens": pt, "max_parts": mp}

    def _prepare(self, batch: Batch, pad_seqs: int = 0, tiles: bool = True):
        ids, qs, ql = batch.arrays()
        pad_tokens = 0
        if tiles and self.gemm_table is not None and batch.num_decode < len(batch.seqs):
            from ..tuning import bucket_rows

            rows = int(np.sum(ql))
            # steps the fused small-prefill path takes (<= SKINNY_MAX_M rows) stay unpadded:
            # its GEMVs read every row of x per weight tile (17 rows padded to 32 doubled
            # gate_up: 80 vs ~40 us)
            if not self.model.small_prefill_ok(rows):
                pad_tokens = bucket_rows(rows)
        d = self.bm.build_batch(ids, qs, ql, self.bt_width,
                                self.tile_tokens if tiles else 0, batch.num_decode, pad_tokens,
                                pad_seqs)
        T = d["positions"].shape[0]
        S = d["seq_kvlen"].shape[0]
        NT = d["tile_seq"].shape[0]
        lay = MetaLayout(T, S, self.bt_width, NT)
        input_ids = np.zeros(T, dtype=np.int32)
        row = 0
        temps = np.zeros(S, dtype=np.float32)
        top_p = np.ones(S, dtype=np.float32)
        top_k = np.zeros(S, dtype=np.int32)
        seeds = np.zeros(S, dtype=np.int64)
        steps = np.zeros(S, dtype=np.int64)
        for i, (seq, s0, n) in enumerate(zip(batch.seqs, batch.q_start, batch.q_len)):
            input_ids[row:row + n] = seq.token_array()[s0:s0 + n]
            row += n
            temps[i] = seq.sampling.temperature
            top_p[i] = seq.sampling.top_p
            top_k[i] = seq.sampling.top_k
            seeds[i] = seq.seed
            steps[i] = len(seq.output_ids)
        arrays = dict(d)
        arrays.update(input_ids=input_ids, temperature=temps, top_p=top_p, top_k=top_k,
                      seeds=seeds, steps=steps, feed_prev=np.zeros(1, dtype=np.int32))
        return lay, arrays

    @property
    def meta_host(self) -> torch.Tensor:
        return self.meta_hosts[self._mh]

    @property
    def meta_host_np(self) -> np.ndarray:
        return self.meta_hosts_np[self._mh]

    def _next_meta_host(self) -> np.ndarray:
        """Switch to the other pinned metadata buffer (waiting for the H2D copy that last
        read it) and return its numpy view."""
        self._mh ^= 1
        ev = self._h2d_done[self._mh]
        if ev is not None:
            ev.synchronize()
        return self.meta_hosts_np[self._mh]

    def _h2d(self, dst: torch.Tensor, size: int):
        dst.copy_(self.meta_host[:size], non_blocking=True)
        ev = self._h2d_done[self._mh]
        if ev is not None:
            ev.record()

    def _pack(self, lay: MetaLayout, arrays: dict) -> np.ndarray:
        host = self._next_meta_host()[:lay.size]
        lay.pack(host, arrays)
        return host

    def _meta(self, v: dict, num_decode: int, num_tiles: int, max_decode_kv: int = 0) -> AttnMeta:
        return AttnMeta(positions=v["positions"], slot_mapping=v["slot_mapping"],
                        block_tables=v["block_tables"], seq_kvlen=v["seq_kvlen"],
                        seq_qstart=v["seq_qstart"], tile_seq=v["tile_seq"],
                        tile_qoff=v["tile_qoff"], logits_idx=v["logits_idx"],
                        num_decode=num_decode, num_tiles=num_tiles, seq_slot=v["seq_slot"],
                        max_decode_kv=max_decode_kv)

    def parts_bucket(self, max_kv: int, batch_size: int = 0) -> int:
        """Smallest partition bucket covering a decode step of ``batch_size`` rows whose
        longest context is max_kv (in the partition size that batch size uses)."""
        pt, top, buckets = self._tier(batch_size)
        need = max(1, math.ceil(max_kv / pt))
        return next((p for p in buckets if p >= need), top)

    def _forward_sample(self, v: dict, md: AttnMeta, num_parts: int, special: bool = False):
        """One step's forward + sampling; ``special``: some row uses top-p / top-k (logits
        are materialised and the top-k / top-p kernel samples every row)."""
        m = self.model
        T = v["input_ids"].shape[0]
        if self.hybrid:
            last = m.forward(v["input_ids"], md, self.cache, rows=v["logits_idx"])
            logits = m.compute_logits(last)
            out = self.ws["tokens"][:logits.shape[0]] if logits.shape[0] <= self.max_seqs else None
            if special:
                return ops.sample_topkp(logits, v["temperature"], v["top_p"], v["top_k"],
                                        v["seeds"], v["steps"], out=out)
            return ops.sample(logits, v["temperature"], v["seeds"], v["steps"], out=out)
        if (self.fused_decode and md.num_tiles == 0
                and md.num_decode == T and m.decode_fusable(T)):
            ws = self._ws_for(T)
            # grid over this step's partition bucket only (num_parts covers every row, in
            # the partition size of this batch size: parts_bucket)
            ws = {**ws, "max_parts": min(num_parts, ws["max_parts"])}
            return m.forward_decode(v["input_ids"], md, self.k_layers, self.v_layers,
                                    ws, v["temperature"], v["seeds"], v["steps"],
                                    prev_tokens=self.ws["tokens"], feed_prev=v["feed_prev"],
                                    top_p=v["top_p"] if special else None, top_k=v["top_k"])
        decode_only = md.num_tiles == 0 and md.num_decode == T
        # final norm on the sampled rows only (each sequence's last token)
        last = m.forward(v["input_ids"], md, self.k_layers, self.v_layers, self.part_out,
                         self.part_lse, num_parts, self.part_tokens,
                         prev_tokens=self.ws["tokens"] if decode_only else None,
                         feed_prev=v["feed_prev"] if decode_only else None,
                         rows=v["logits_idx"])
        if not special and m.decode_fusable(last.shape[0]) and \
                last.shape[0] <= self.max_seqs and m.hidden_fusable():
            # fused LM head + Gumbel-max sampler on the (already normalised) last rows
            return m.sample_rows(last, 0.0, v["temperature"], v["seeds"], v["steps"], self.ws)
        logits = m.compute_logits(last)
        # decode-only steps sample straight into ws["tokens"]: a graph replay (and the next
        # look-ahead step's embed) reads the samples from there, so the captured sampler must
        # write them there too (a fresh tensor would leave the previous step's tokens behind)
        out = self.ws["tokens"][:logits.shape[0]] if decode_only else None
        if special:
            return ops.sample_topkp(logits, v["temperature"], v["top_p"], v["top_k"],
                                    v["seeds"], v["steps"], out=out)
        return ops.sample(logits, v["temperature"], v["seeds"], v["steps"], out=out)

    # ------------------------------------------------------------------------------------
    def _graph_ok(self, bucket: int, special: bool = False) -> bool:
        """Can a decode step of this bucket be captured?  Every collective inside it must be
        device-side: RCCL, or - on a gloo control group (TP ranks rehearsing on one GPU) - the
        IPC kernels, which carry the fused decode step's X1/X2 sums and X4 key MAX but not the
        logits all-gather of the top-k / top-p sampler or of buckets past the fused path."""
        c = self.comm
        if c is None or c.size == 1 or not c.is_gloo:
            return True
        return (c.decode_capturable and not special and self.fused_decode
                and self.model.decode_fusable(bucket))

    def graph_bucket(self, batch: Batch) -> int:
        """Graph bucket a decode-only batch replays from (0: eager step)."""
        n = len(batch.seqs)
        if not (self.is_cuda and self.cfg.use_graphs and batch.num_decode == n and n > 0
                and self.graph_sizes and n <= self.graph_sizes[-1]):
            return 0
        b = next(b for b in self.graph_sizes if b >= n)
        return b if self._graph_ok(b, self._special(batch)) else 0

    @staticmethod
    def _special(batch: Batch) -> bool:
        return any(s.sampling.top_p < 1.0 or s.sampling.top_k > 0 for s in batch.seqs)

    def execute(self, batch: Batch) -> np.ndarray:
        """Run one step; returns sampled token ids (one per sequence in batch order)."""
        n = len(batch.seqs)
        bucket = self.graph_bucket(batch)
        if bucket:
            return self.collect(self.launch(batch))
        self.steps += 1
        special = self._special(batch)
        lay, arrays = self._prepare(batch)
        max_kv = int(arrays["seq_kvlen"][:batch.num_decode].max()) if batch.num_decode else 0
        if batch.num_decode == n and lay.NT == 0:
            # decode-only: in the partition size of this batch size (>= the 256-token count
            # the unfused path needs, within the allocated partials)
            num_parts = self.parts_bucket(max_kv, n)
        else:
            num_parts = max(1, math.ceil(max_kv / self.part_tokens))
        host = self._pack(lay, arrays)
        hdr = np.array([OP_STEP, lay.T, lay.S, lay.W, lay.NT, batch.num_decode, num_parts,
                        0, int(special), n, lay.size, max_kv], dtype=np.int32)
        if self.publisher is not None:
            self.publisher.publish(np.concatenate([hdr, host]))
        toks = self._run(hdr)
        if self.is_cuda and lay.T > n and not self.hybrid and \
                self.model.prefill_gemm != "hipblaslt":
            # prefill rows ran: fetch the hand-written GEMM's error word with the tokens'
            # own sync (a cross-workgroup wait that timed out - outputs are still exact, the
            # workgroup recomputed; it signals a GPU shared with other work) - ADVICE r3
            self._err_host.zero_()
            ops.prefill_gemm_error_to(self._err_host, clear=True)
        out = toks[:n].cpu().numpy()
        word = int(self._err_host[0]) if self.is_cuda else 0
        if word:
            self._err_host.zero_()
            with self._kernel_error_lock:
                self.kernel_error |= word
                self.kernel_error_steps += 1
            print(f"[model_runner] prefill GEMM error word {word:#x}: a "
                  "cross-workgroup wait timed out (tiles recomputed, outputs exact; the GPU "
                  "is shared or oversubscribed)", flush=True)
        return out

    def execute_logits(self, batch: Batch, rows, layer_out=None) -> np.ndarray:
        """Run one step without sampling and return the fp32 logits [len(rows), vocab] of the
        given rows of the step (row r = r-th token of the batch in sequence order).  The step
        advances the cache and the state exactly as ``execute`` does: it is the same forward
        with another set of output rows (trace replay, evaluation)."""
        self.steps += 1
        lay, arrays = self._prepare(batch)
        max_kv = int(arrays["seq_kvlen"][:batch.num_decode].max()) if batch.num_decode else 0
        num_parts = max(1, math.ceil(max_kv / getattr(self, "part_tokens", 256)))
        self._pack(lay, arrays)
        dev = self.meta_dev[:lay.size]
        self._h2d(dev, lay.size)
        v = lay.views(dev)
        md = self._meta(v, batch.num_decode, lay.NT, max_kv)
        rows_t = torch.as_tensor(np.asarray(rows, dtype=np.int64)).to(self.device)
        if rows_t.numel() == 0:
            rows_t = torch.zeros(1, dtype=torch.int64, device=self.device)
        if self.hybrid:
            hidden = self.model.forward(v["input_ids"], md, self.cache, rows=rows_t,
                                        layer_out=layer_out)
        else:
            if self.publisher is not None:
                raise RuntimeError("execute_logits runs on a single rank")
            hidden = self.model.forward(v["input_ids"], md, self.k_layers, self.v_layers,
                                        self.part_out, self.part_lse, num_parts, self.part_tokens,
                                        rows=rows_t)
        logits = self.model.compute_logits(hidden).float()
        return logits[:len(rows)].cpu().numpy()

    def take_kernel_error(self) -> int:
        """Error words seen since the previous call (the /health check), then cleared."""
        with self._kernel_error_lock:
            w, self.kernel_error = self.kernel_error, 0
        return w

    def launchable(self, batch: Batch) -> bool:
        """Decode-only batches can be launched asynchronously (every sampler runs on the
        device and leaves its tokens in ws["tokens"])."""
        # (hybrid models read their input tokens from the step's metadata: no look-ahead)
        return not self.hybrid and self._decode_only(batch)

    def _decode_only(self, batch: Batch) -> bool:
        n = len(batch.seqs)
        return 0 < n <= self.max_seqs and batch.num_decode == n

    def launch(self, batch: Batch, lookahead: bool = False) -> dict:
        """Enqueue one decode-only step (graph replay when a bucket fits, else eager) and its
        token D2H copy; returns a handle for ``collect``.  ``lookahead``: the batch continues
        the previous launch row for row and its input tokens are that step's device samples
        (``ws["tokens"]``, not yet seen by the host), so the host never waits between steps
        (async look-ahead decode)."""
        if not self._decode_only(batch):
            raise ValueError("launch() needs a decode-only batch")
        n = len(batch.seqs)
        bucket = self.graph_bucket(batch)
        special = int(self._special(batch))
        self.steps += 1
        t0 = time.perf_counter()
        if bucket:
            lay, arrays = self._prepare(batch, pad_seqs=bucket, tiles=False)
            num_parts = self.parts_bucket(int(arrays["seq_kvlen"][:n].max()), bucket)
            if (bucket, num_parts, special) not in self.graphs:
                self.capture(bucket, num_parts, bool(special))
                t0 = time.perf_counter()
            assert lay.size == self.graph_io[(bucket, num_parts, special)]["layout"].size
        else:
            lay, arrays = self._prepare(batch, tiles=False)
            num_parts = self.parts_bucket(int(arrays["seq_kvlen"][:n].max()), n)
        arrays["feed_prev"] = np.array([1 if lookahead else 0], dtype=np.int32)
        host = self._pack(lay, arrays)
        hdr = np.array([OP_STEP, lay.T, lay.S, lay.W, lay.NT, batch.num_decode, num_parts,
                        bucket, special, n, lay.size, 0], dtype=np.int32)
        if self.publisher is not None:
            self.publisher.publish(np.concatenate([hdr, host]))
        t1 = time.perf_counter()
        self._run(hdr)
        dev_toks = self.ws["tokens"]  # _run leaves decode samples here (graph or eager)
        slot = self._mh  # one token slot per metadata buffer: same reuse distance
        ev = self._tok_done[slot]
        if ev is not None:
            ev.synchronize()
        self.tok_host[slot][:n].copy_(dev_toks[:n], non_blocking=self.is_cuda)
        if ev is not None:
            ev.record()
        if bucket:
            self.timing["graph_prep"] += t1 - t0
        return {"n": n, "slot": slot, "t_launch": t1, "graph": bool(bucket)}

    def collect(self, h: dict) -> np.ndarray:
        """Wait for a launched step's tokens."""
        ev = self._tok_done[h["slot"]]
        if ev is not None:
            ev.synchronize()
        now = time.perf_counter()
        if h["graph"]:
            # pipelined steps overlap: charge each step from the later of its launch and the
            # previous collect, so graph_run / graph_steps stays the per-step wall time
            self.timing["graph_run"] += now - max(h["t_launch"], self._last_collect)
        self._last_collect = now
        return self.tok_host[h["slot"]][:h["n"]].numpy().copy()

    def _run(self, hdr):
        """Execute one step from its header; the packed metadata is in ``meta_host``."""
        T, S, W, NT, num_decode, num_parts, bucket, special, n, size = (int(x) for x in hdr[1:11])
        max_kv = int(hdr[11])  # longest decode context of the step (eager steps)
        if bucket:
            key = (bucket, num_parts, special)
            io = self.graph_io[key]
            self._h2d(io["dev"], size)
            self.graphs[key].replay()
            self.graph_steps += 1
            return io["out"]
        lay = MetaLayout(T, S, W, NT)
        dev = self.meta_dev[:size]
        self._h2d(dev, size)
        v = lay.views(dev)
        md = self._meta(v, num_decode, NT, max_kv)
        # every rank samples (deterministic kernels over all-gathered logits under TP)
        out = self._forward_sample(v, md, num_parts, bool(special))
        if NT == 0 and num_decode == T and out is not None:
            # every rank keeps the decode samples where a look-ahead step embeds them from
            dev_toks = self.ws["tokens"]
            if out.data_ptr() != dev_toks.data_ptr():
                dev_toks[:T].copy_(out[:T])
        return out

    # -- TP worker side ------------------------------------------------------------------
    def serve_worker(self, channel, reader: int) -> None:
        """TP rank > 0: replay rank 0's steps until it publishes OP_STOP / closes.

        Liveness: the worker registers its pid on the channel (rank 0 fails its next publish
        naming a dead worker) and waits in 1 s slices, raising when rank 0's process is gone
        so an orphaned worker exits instead of holding its GPU forever."""
        last = 0
        if hasattr(channel, "register_reader"):
            channel.register_reader(reader)
        while True:
            msg = channel.receive(reader, last, 1.0)
            if msg is None:
                if channel.closed:
                    return
                if not getattr(channel, "writer_alive", True):
                    raise RuntimeError(f"TP rank {reader + 1}: rank 0 died; worker exiting")
                continue
            last, data = msg
            hdr = data[:HDR_WORDS]
            op = int(hdr[0])
            if op == OP_STOP:
                return
            if op == OP_CAPTURE:
                self.capture(int(hdr[1]), int(hdr[2]) or None, bool(hdr[3]))
                continue
            if op == OP_BARRIER:
                if self.is_cuda:
                    torch.cuda.synchronize(self.device)
                self.comm.barrier()
                continue
            size = int(hdr[10])
            # alternate pinned buffers: no stream sync per step, only an event wait on the
            # copy two steps back before its buffer is rewritten
            self._next_meta_host()[:size] = data[HDR_WORDS:HDR_WORDS + size]
            self._run(hdr)
            self.steps += 1

    def barrier(self):
        """Synchronise every TP rank (device work drained, then a process-group barrier)."""
        if self.is_cuda:
            torch.cuda.synchronize(self.device)
        if self.publisher is not None:
            hdr = np.zeros(HDR_WORDS, dtype=np.int32)
            hdr[0] = OP_BARRIER
            self.publisher.publish(hdr)
        if self.comm is not None:
            self.comm.barrier()

    def stop_workers(self):
        if self.publisher is not None:
            hdr = np.zeros(HDR_WORDS, dtype=np.int32)
            hdr[0] = OP_STOP
            try:
                self.publisher.publish(hdr, 30.0)
            finally:
                self.publisher.close()

    # ------------------------------------------------------------------------------------
    def capture(self, bucket: int, parts: int | None = None, special: bool = False):
        """Capture a decode step for `bucket` sequences whose contexts fit `parts` attention
        partitions (default: max_model_len) into a hipGraph; ``special``: the top-k / top-p
        sampler variant (logits materialised)."""
        parts = parts or self._tier(bucket)[1]
        if self.publisher is not None:
            hdr = np.zeros(HDR_WORDS, dtype=np.int32)
            hdr[0], hdr[1], hdr[2], hdr[3] = OP_CAPTURE, bucket, parts, int(special)
            self.publisher.publish(hdr)
        lay = MetaLayout(bucket, bucket, self.bt_width, 0)
        dev = torch.zeros(lay.size, dtype=torch.int32, device=self.device)
        v = lay.views(dev)
        # dummy sequences: kvlen 0, slot -1 -> kernels skip them
        v["seq_qstart"].copy_(torch.arange(bucket + 1, dtype=torch.int32))
        v["slot_mapping"].fill_(-1)
        v["logits_idx"].copy_(torch.arange(bucket, dtype=torch.int64))
        if self.hybrid:
            # dummy sequences own no state slot: the warm-up passes below must not touch slot 0
            v["seq_slot"].fill_(-1)
        md = self._meta(v, bucket, 0, parts * self.part_tokens)
        # a capture may come between look-ahead steps (a new partition bucket mid-generation):
        # the warm-up passes sample into ws["tokens"], which still holds the in-flight step's
        # tokens the next step embeds - keep them (stream-ordered copy and restore)
        saved_tokens = self.ws["tokens"].clone()
        stream = torch.cuda.Stream(self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            for _ in range(2):  # warm up (hipBLASLt heuristics, allocator)
                self._forward_sample(v, md, parts, special)
        torch.cuda.current_stream(self.device).wait_stream(stream)
        dump_dir = os.environ.get("ATTA_GRAPH_DUMP_DIR")
        # node-level dump of every captured step (scripts/gpu/graph_nodes.py) keeps the
        # hipGraph after instantiation so its nodes can be listed
        g = torch.cuda.CUDAGraph(keep_graph=True) if dump_dir else torch.cuda.CUDAGraph()
        if self.graph_pool is None:
            self.graph_pool = torch.cuda.graph_pool_handle()
        with torch.cuda.graph(g, pool=self.graph_pool, stream=stream):
            out = self._forward_sample(v, md, parts, special)
            toks = self.ws["tokens"]
            if out.data_ptr() != toks.data_ptr():  # every sampler path ends in ws["tokens"]
                toks[:bucket].copy_(out[:bucket])
                out = toks[:bucket]
        self.ws["tokens"].copy_(saved_tokens)
        torch.cuda.synchronize(self.device)
        key = (bucket, parts, int(special))
        if dump_dir:
            os.makedirs(dump_dir, exist_ok=True)
            nodes = ops._native().graph_nodes(int(g.raw_cuda_graph()))
            path = os.path.join(dump_dir, f"tp{self.tp_size}_rank{self.tp_rank}_b{bucket}"
                                          f"_p{parts}_s{int(special)}.nodes")
            with open(path, "w") as f:
                f.write("\n".join(nodes) + "\n")
        self.graphs[key] = g
        self.graph_io[key] = {"layout": lay, "dev": dev, "out": out}

    def capture_all(self, all_parts: bool = False):
        """Capture every batch bucket at the full partition count (shorter-context partition
        buckets are captured on first use, or here with ``all_parts``)."""
        if not (self.is_cuda and self.cfg.use_graphs):
            return
        for b in self.graph_sizes:
            if not self._graph_ok(b):
                continue
            _, top, buckets = self._tier(b)
            for p in (buckets if all_parts else [top]):
                if (b, p, 0) not in self.graphs:
                    self.capture(b, p)

    def warm_library_gemms(self) -> int:
        """Run every shape of the loaded TunableOp table that this rank's weights have once
        (bf16: plain and residual-add GEMM; fp8: the row-scaled GEMM), so each rocBLAS /
        hipBLASLt solution's code object - and the libraries themselves - load at engine
        start, not inside the first request of that bucket (rocBLAS initialisation alone put
        ~1.1 s into the first 560-row prefill, bench/coldstart.py).  Returns the GEMMs run."""
        if self.gemm_table is None or not self.is_cuda or not self.model.layers:
            return 0
        import re

        L = self.model.layers[0]
        ws = {}
        for name in ("qkv", "o", "gate_up", "down"):
            w = getattr(L, name)
            ws[tuple(w.shape)] = (w, getattr(L, name + "_s"))
        ws.setdefault(tuple(self.model.lm_head.shape), (self.model.lm_head, None))
        pat = re.compile(r"^(\w+?)_TN,tn_(\d+)_(\d+)_(\d+)_")
        n = 0
        with open(self.gemm_table) as f, torch.inference_mode():
            for line in f:
                mt = pat.match(line)
                if mt is None:
                    continue
                op, N, M, K = mt.group(1), int(mt.group(2)), int(mt.group(3)), int(mt.group(4))
                w, s = ws.get((N, K), (None, None))
                if w is None:
                    continue
                if op.startswith("ScaledGemm") and s is not None:
                    xq = torch.zeros(M, K, dtype=torch.uint8, device=self.device)
                    ops.gemm_fp8(xq, torch.ones(M, 1, device=self.device), w, s, self.dtype)
                elif op.startswith("GemmTunableOp") and s is None and w.dtype == self.dtype:
                    x = torch.zeros(M, K, dtype=w.dtype, device=self.device)
                    torch.nn.functional.linear(x, w)
                    torch.zeros(M, N, dtype=w.dtype, device=self.device).addmm_(x, w.t())
                else:
                    continue
                n += 1
        torch.cuda.synchronize(self.device)
        return n

    def reset_state(self):
        """Drop prefix cache contents (used between benchmark phases)."""
        self.bm.reset_prefix_cache()


__all__ = ["ModelRunner", "MetaLayout", "ref", "HDR_WORDS", "OP_STEP", "OP_CAPTURE", "OP_STOP",
           "OP_BARRIER"]
