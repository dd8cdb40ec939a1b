"""Per-GPU rendezvous of the K virtual stream workers (VSWs) around one fused launch.

In IIDP every VSW runs its own DDP reducer on its own thread and stream; only VSW 0's
comm hook communicates, the others register ``dummy_hook``
(jabas/train/trainer.py:452-468). ``LocalBucketSync`` is where those K hooks meet on one
GPU: each hook publishes the flat bucket it was handed; when the K buckets with the same
index are in, whichever thread arrived last queues ONE fused kernel on VSW 0's stream
(aggregate into VSW 0's bucket, statistics when asked, optimizer update when the weights
are laid out like the buckets). The Future a hook gets back is already complete: stock
DDP waits on it at the end of that replica's backward on the autograd engine's device
thread, which every replica on the GPU shares, so a Future that needed another replica's
backward to make progress would deadlock. Ordering is by stream instead: the launch waits
on an event from every VSW's stream, and ``finish_step`` makes every VSW stream wait for
the launches (and reports anything that went wrong in them) before gradients are reused.
"""
import threading

import torch

from . import sync
from . import _lib as L


class BucketStats:
    """Statistics row of one bucket on the device (what a stat step leaves in
    ``GradientSimilarityState.grad_placeholder`` instead of a full gradient copy). The row is
    one of two buffers the bucket's launches alternate between: read it (``cpu()``) before the
    second-next statistic step of that bucket."""

    def __init__(self, index, row):
        self.index, self.row = index, row

    def cpu(self):
        return self.row.detach().to("cpu")


class _Slot:
    def __init__(self, K):
        self.tensors = [None] * K
        self.events = [None] * K
        self.want_stats = False
        self.on_done = None
        self.count = 0


class LocalBucketSync:
    """batches: local batch size of each VSW on this GPU (defines K and the weights).

    launcher(bucket_index, tensors, want_stats) -> stats row or None replaces the C-ABI
    call (CPU tests of the protocol inject a recorder); the default queues
    ``jabas_sync_bucket`` on VSW 0's stream.
    """

    def __init__(self, batches, launcher=None, opt=None, param_buckets=None, deferred=False):
        """deferred: collect the buckets of a step and queue ONE planned launch over all of them in
        ``finish_step`` instead of one launch per bucket as each becomes complete. The per-bucket mode
        overlaps the sync with the rest of the backward pass; the deferred mode spends less GPU time
        (one ramp-up and drain: 0.68 ms against 0.9 ms wall for the 14 buckets of ViT-B/16) and less host
        time, and the buckets hold the aggregate only after ``finish_step``."""
        if deferred and launcher is not None:
            raise ValueError("the deferred mode drives the C ABI itself: no launcher can be injected")
        self.deferred = bool(deferred)
        self._ready = {}                       # deferred mode: bucket index -> complete _Slot of this step
        self._vsw_streams = {}                 # deferred mode: VSW index -> the stream its hooks ran on
        self._plan = self._plan_key = None
        self.batches = tuple(batches)
        self.K = len(self.batches)
        self.opt = opt
        self.param_buckets = param_buckets or {}     # bucket index -> dict(param=, state1=, state2=, bounds=, fanout=)
        self.step_count = 0
        self.lr_scale = 1.0
        self.accumulations = 1                 # micro-batches each VSW summed into its buckets (no_sync() steps + 1)
        self._launcher = launcher or self._launch_fused
        self._lock = threading.Lock()
        self._slots = {}
        self._main_stream = None
        self._calls = {}                       # bucket index -> prepared sync.BucketCall
        self._args_cache = {}
        self._launch_streams = set()           # streams that carry launches of the current step
        self._errors = []
        self.launched = 0                      # fused launches queued so far

    # ------------------------------------------------------------------ hooks call this
    def publish(self, k, bucket_index, tensor, want_stats=False, on_done=None, value=None):
        """Hands VSW k's bucket ``bucket_index`` over; the fused launch for that bucket is
        queued by whichever VSW hands its bucket over last. Returns a completed Future
        carrying ``value`` (default the tensor)."""
        if not 0 <= k < self.K:
            raise ValueError(f"VSW index {k} outside 0..{self.K - 1}")
        fut = torch.futures.Future()
        fut.set_result(tensor if value is None else value)
        event = stream = None
        if tensor.is_cuda:
            stream = torch.cuda.current_stream(tensor.device)
            if self.deferred:                  # ordered once per VSW stream in finish_step, not once per bucket
                self._vsw_streams[k] = stream
            elif k != 0:                       # VSW 0's stream is the one the launch is queued on
                event = torch.cuda.Event()
                event.record(stream)
        with self._lock:
            slot = self._slots.setdefault(bucket_index, _Slot(self.K))
            if slot.tensors[k] is not None:
                raise RuntimeError(f"VSW {k} published bucket {bucket_index} twice in one step")
            slot.tensors[k], slot.events[k] = tensor, event
            slot.count += 1
            if k == 0:
                slot.want_stats, slot.on_done = want_stats, on_done
                self._main_stream = stream
            ready = slot.count == self.K
            if ready:
                del self._slots[bucket_index]
        if ready:
            if self.deferred:
                with self._lock:
                    self._ready[bucket_index] = slot
            else:
                self._fire(bucket_index, slot)
        return fut

    def _fire(self, bucket_index, slot):
        main = self._main_stream
        try:
            if main is not None:
                for ev in slot.events[1:]:
                    main.wait_event(ev)
                row = self._launcher(bucket_index, slot.tensors, slot.want_stats)
                self._launch_streams.add(main)
            else:
                row = self._launcher(bucket_index, slot.tensors, slot.want_stats)
        except Exception as exc:                       # reported by finish_step
            with self._lock:
                self._errors.append((bucket_index, exc))
            return
        if slot.on_done is not None:
            slot.on_done(BucketStats(bucket_index, row) if row is not None else None)
        with self._lock:
            self.launched += 1

    # ------------------------------------------------------------- the default launcher
    def _step_args(self, dtype, want_stats, with_opt):
        """JabasStepArgs of this step, built once per (step, kind of launch) and shared by its buckets."""
        key = (self.step_count, self.lr_scale, self.accumulations, dtype, bool(want_stats), bool(with_opt))
        hit = self._args_cache.get(key)
        if hit is None:
            if len(self._args_cache) > 8:
                self._args_cache.clear()
            hit = self._args_cache[key] = sync.make_step_args(
                self.batches, dtype, stats=want_stats, opt=self.opt if with_opt else None,
                step=self.step_count + 1, first_step=self.step_count == 0, lr_scale=self.lr_scale,
                accumulations=self.accumulations)
        return hit

    def _launch_fused(self, bucket_index, tensors, want_stats):
        """Queues ``jabas_sync_bucket`` for one bucket on VSW 0's stream. DDP hands a hook the same
        bucket buffers every step, so the prepared call (validated span, C struct, device bound table,
        workspace) is kept per bucket and rebuilt only when the buffers change."""
        call = self._calls.get(bucket_index)
        if call is None or not call.matches(tensors):
            span, with_opt = self._span_of(bucket_index, tensors)
            call = self._calls[bucket_index] = sync.BucketCall(span)
            call.with_opt = with_opt
        args = self._step_args(tensors[0].dtype, want_stats, call.with_opt)
        return call.run(args, stream=self._main_stream)

    def _span_of(self, bucket_index, tensors):
        """(span over the K buffers of one bucket, whether the optimizer runs in the same launch)."""
        g0 = tensors[0]
        pb = self.param_buckets.get(bucket_index)
        opt = self.opt if pb is not None else None
        span = sync.SpanSpec(tensors, agg_out=g0 if g0.dtype == torch.float32 else (pb or {}).get("agg_out"),
                             param=pb and pb.get("param"), state1=pb and pb.get("state1"),
                             state2=pb and pb.get("state2"), fanout=(pb or {}).get("fanout", ()),
                             bounds=(pb or {}).get("bounds", ()) if opt else ())
        return span, opt is not None

    def _fire_all(self):
        """Deferred mode: one planned launch over every bucket of the step, in bucket order."""
        with self._lock:
            ready, self._ready = self._ready, {}
        order = sorted(ready)
        slots = [ready[i] for i in order]
        with_opt = [self.opt is not None and i in self.param_buckets for i in order]
        main = self._main_stream
        if main is None or (any(with_opt) and not all(with_opt)):
            for i, slot in zip(order, slots):          # host tensors (protocol tests), or buckets with and without
                self._fire(i, slot)                    # weights behind them: one launch each after all
            return
        try:
            # everything the other VSWs queued up to now (their whole backward) precedes the launch: one
            # event per stream instead of one per bucket and VSW, which on the GPU's queue are a barrier
            # packet each (98 of them per step for 14 buckets x 4 VSWs cost 0.25 ms)
            for k, stream in sorted(self._vsw_streams.items()):
                if k != 0 and stream != main:
                    ev = torch.cuda.Event()
                    ev.record(stream)
                    main.wait_event(ev)
            key = tuple((i, slot.tensors[0].numel()) + tuple(t.data_ptr() for t in slot.tensors)
                        for i, slot in zip(order, slots))
            if key != self._plan_key:                   # DDP hands over the same buffers every step: built once
                spans = [self._span_of(i, slot.tensors)[0] for i, slot in zip(order, slots)]
                self._plan = sync.SyncPlan(spans, sync.opt_kind(self.opt) if with_opt[0] else L.OPT_NONE)
                self._plan_key = key
            want = any(slot.want_stats for slot in slots)
            args = self._step_args(slots[0].tensors[0].dtype, want, with_opt[0])
            rows = self._plan.run(args, stream=main)
            if rows is not None:
                with torch.cuda.stream(main):
                    rows = rows.clone()                 # the plan's own rows are overwritten by its next launch
            self._launch_streams.add(main)
        except Exception as exc:
            with self._lock:
                self._errors.append((order[0], exc))
            return
        for j, (i, slot) in enumerate(zip(order, slots)):
            if slot.on_done is not None:
                slot.on_done(BucketStats(i, rows[j]) if slot.want_stats and rows is not None else None)
        with self._lock:
            self.launched += 1

    # ------------------------------------------------------------------ trainer calls this
    def pending(self):
        with self._lock:
            return sorted(self._slots)

    def finish_step(self, streams=()):
        """End of a sync step: every VSW stream waits for the fused launches that read its
        buckets, and the step count (Adam's t, SGD's first-step flag) advances."""
        left = self.pending()
        if left:
            raise RuntimeError(f"buckets {left} were not published by every VSW")
        if self._ready:
            self._fire_all()
        # the launches of a step sit on VSW 0's stream in order: one event behind the last of them orders
        # every VSW stream behind all of them
        launch_streams, self._launch_streams = self._launch_streams, set()
        for main in launch_streams:
            done = torch.cuda.Event()
            done.record(main)
            for s in streams:
                if s != main:
                    s.wait_event(done)
        with self._lock:
            errors, self._errors = self._errors, []
        if errors:
            idx, exc = errors[0]
            raise RuntimeError(f"fused launch of bucket {idx} failed: {exc}") from exc
        self.step_count += 1
