"""PyTorch modules around the fused embedding kernel.

Class names, constructor arguments and ``forward`` signatures follow
``RecFlex/rec_modules.py:19-179`` (``FeatPreprocess``, ``FeatEmbed``, ``FeatProcessEmbed``,
``RecomModel``), so code written against the reference keeps working:

* ``FeatPreprocess.forward(raw_data, max_concurrent_blocks)`` parses the sample lines on the
  CPU and returns the 9-tuple ``(arg_buffers, data_buffer_offsets, scala_args, extra_buffers,
  extra_buffer_offsets, task_mapping, task_tiles, task_barriers, output_size)``;
* ``FeatEmbed.forward(*that tuple, timing=False, timing_schedules=None)`` runs the fused kernel
  and returns the flat fp32 output of ``output_size / 4`` elements (reshape to
  ``[-1, output_units]``), or ``(output, task_times)`` with ``timing=True``;
* ``FeatEmbed.forward_indices(indices, offsets)`` is the tensor entry point (per-feature int32
  device tensors in, ``[batch, sum(dim)]`` out) that the reference does not have.

Differences from the reference: the kernel library is a ``RecomLib`` (ctypes handle on a
generated ``librecom.so``) instead of process-global ``torch.ops.recom``; thread binding happens
on the GPU, so ``task_mapping`` / ``task_tiles`` / ``task_barriers`` / ``extra_buffers`` are
accepted and ignored; tables may be fp32, fp16 or row-wise int8; the kernel runs on torch's
current stream.  There is no CPU fallback: without a built library the modules raise.
"""

from typing import List, NamedTuple, Optional, Sequence, Tuple, Union

import numpy as np
import torch
import torch.nn as nn

from .librecom import RecomLib
from .quant import random_int8_table

_current_lib: Optional[RecomLib] = None

_TORCH_DTYPES = {0: torch.float32, 1: torch.float16, 2: torch.uint8}


def load_library(librecom_path: str) -> RecomLib:
    """Counterpart of ``torch.ops.load_library(librecom_path)`` (rec_modules.py:122-123):
    makes the library the default for modules constructed afterwards."""
    global _current_lib
    _current_lib = RecomLib(librecom_path)
    return _current_lib


def _resolve_lib(librecom: Union[None, str, RecomLib]) -> RecomLib:
    if isinstance(librecom, RecomLib):
        return librecom
    if isinstance(librecom, str):
        return RecomLib(librecom)
    if _current_lib is None:
        raise RuntimeError("no fused-kernel library loaded: pass librecom=... or call "
                           "recflex_amd.rec_modules.load_library(path) first")
    return _current_lib


class FeatPreprocess(nn.Module):
    def __init__(self, recom_host, device: torch.device, output_units: int = None):
        super(FeatPreprocess, self).__init__()
        self.recom_host = recom_host
        self.device = device
        self.output_units = output_units

    def forward(self, raw_data: List[List[str]], max_concurrent_blocks: int = 0):
        (data_buffer_offsets, output_offsets, extra_buffer_offsets, task_mapping, task_tiles,
         data, scala_data) = self.recom_host.preprocess(raw_data, max_concurrent_blocks)

        output_size: int = output_offsets[-1]
        if output_size == 0 and self.output_units and len(raw_data) > 0:
            output_size = len(raw_data[0]) * self.output_units * 4
        total_blocks = len(task_mapping)

        extra_buffers = torch.empty([extra_buffer_offsets[-1]], dtype=torch.int8, device=self.device)
        task_barriers = torch.zeros([total_blocks], dtype=torch.int32, device=self.device)

        packed = getattr(self.recom_host, "packed", None)
        if packed is None:
            packed = np.concatenate([np.asarray(d, dtype=np.int32) for d in data]) if data \
                else np.zeros(0, np.int32)
        arg_buffers = torch.from_numpy(packed).to(self.device)
        data_buffer_offsets = torch.tensor(data_buffer_offsets, dtype=torch.int64, device=self.device)
        extra_buffer_offsets = torch.tensor(extra_buffer_offsets, dtype=torch.int32, device=self.device)
        task_mapping = torch.tensor(task_mapping, dtype=torch.int32, device=self.device).reshape(-1, 2)
        task_tiles = torch.tensor(task_tiles, dtype=torch.int32, device=self.device)
        scala_args = torch.tensor(scala_data, dtype=torch.int32, device=self.device)

        return (
            arg_buffers,
            data_buffer_offsets,
            scala_args,
            extra_buffers,
            extra_buffer_offsets,
            task_mapping,
            task_tiles,
            task_barriers,
            output_size,
        )


class FeatEmbed(nn.Module):
    def __init__(self, device: torch.device, embed_tables: List[torch.Tensor] = None,
                 table_shapes: List[Tuple[int, int]] = None,
                 librecom: Union[None, str, RecomLib] = None):
        super(FeatEmbed, self).__init__()
        self.device = torch.device(device) if not isinstance(device, int) else torch.device("cuda", device)
        self.lib = _resolve_lib(librecom)

        if embed_tables:
            self.embed_tables = list(embed_tables)
        elif table_shapes:
            self.embed_tables = []
            for f, (rows, dim) in enumerate(table_shapes):
                dt = self.lib.dtypes[f] if f < self.lib.num_features else 0
                if dt == 2:
                    table = random_int8_table(rows, dim, self.device)
                else:
                    table = torch.randn((rows, dim), dtype=torch.float32, device=self.device)
                    if dt == 1:
                        table = table.half()
                self.embed_tables.append(table)
        else:
            raise Exception("At least one of embed_tables and table_shapes should be given!")
        self._check_tables()

        # address of each table (reference: torch.ops.recom.get_gpu_pointers_array)
        self.embed_table_ptrs = torch.tensor([t.data_ptr() for t in self.embed_tables],
                                             dtype=torch.int64, device=self.device)
        self.max_concurrent_blocks = self.lib.get_max_concurrent_blocks()

        # Workspace of the split-bag schedules (partial sums and arrival counters of bags summed
        # by several workgroups): zeroed once, every launch leaves the counters at zero again.
        # It has the role of the reference's extra_buffers / task_barriers
        # (RecFlex/rec_modules.py:44-52), allocated per module instead of per batch; launches of
        # one module must not overlap on different streams.
        self.workspace = None
        if self.lib.workspace_bytes:
            self.workspace = torch.zeros((self.lib.workspace_bytes + 3) // 4, dtype=torch.int32,
                                         device=self.device)
            torch.cuda.synchronize(self.device)

        self.output_units = self.lib.embed_dim_sum
        # timing builds: (time before the first tile, time in all) summed over the workgroups of
        # the last timed launch, in units of 10 ns (the constant 100 MHz clock)
        self.last_workgroup_ticks = None
        self._io_cache_key = None
        self._io_bound = None

    def _check_tables(self) -> None:
        lib = self.lib
        if len(self.embed_tables) != lib.num_features:
            raise ValueError(f"library was emitted for {lib.num_features} features, "
                             f"got {len(self.embed_tables)} tables")
        for f, t in enumerate(self.embed_tables):
            want = _TORCH_DTYPES[lib.dtypes[f]]
            cols = lib.row_strides[f] if lib.dtypes[f] == 2 else lib.embed_dims[f]
            if t.dtype != want or t.dim() != 2 or t.shape[1] != cols:
                raise ValueError(f"table {f}: expected [rows, {cols}] {want}, got {list(t.shape)} {t.dtype}")
            if not t.is_contiguous():
                raise ValueError(f"table {f} is not contiguous")
            if t.device.type != "cuda":
                raise ValueError(f"table {f} is on {t.device}; the fused kernel needs device memory")
            if t.data_ptr() % 16 != 0:
                raise ValueError(f"table {f} is not 16-byte aligned")

    # -------------------------------------------------------------------------------------

    def _launch(self, batch: int, timing: bool, timing_schedules: Optional[int], tile_bytes: int,
                grid_blocks: int, schedule_choice: torch.Tensor = None, out: torch.Tensor = None,
                xcd_segments: int = 0, kernel_events=None, **inputs):
        row_stride = 0
        if out is not None:
            if out.dtype != torch.float32 or out.numel() != batch * self.output_units \
                    or out.device.type != "cuda":
                raise TypeError(f"out must be an fp32 device tensor of "
                                f"{batch * self.output_units} elements")
            if out.is_contiguous():
                output = out.view(-1)
            elif out.dim() == 2 and out.shape == (batch, self.output_units) and out.stride(1) == 1:
                # a column slab of a wider buffer: the library writes rows out.stride(0) apart
                output, row_stride = out, out.stride(0)
            else:
                raise TypeError("out must be contiguous, or a [batch, sum(dim)] view with unit "
                                "column stride (a column slab of a wider buffer)")
        else:
            output = torch.empty([batch * self.output_units], dtype=torch.float32, device=self.device)
        times = None
        if timing:
            if not self.lib.info.timing:
                raise RuntimeError("timing=True needs a library emitted with timing=True")
            # per-feature ticks (shader cycles), then the workgroups' time before their first
            # tile and all of their time in units of 10 ns (kept in self.last_workgroup_ticks)
            times = torch.zeros([self.lib.num_features + 2], dtype=torch.int64, device=self.device)
        if schedule_choice is not None:
            if schedule_choice.dtype != torch.int32 or schedule_choice.numel() != len(self.embed_tables) \
                    or schedule_choice.device.type != "cuda":
                raise TypeError("schedule_choice must be an int32 device tensor with one entry per feature")
            inputs["schedule_choice"] = schedule_choice.data_ptr()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        if kernel_events is not None:
            inputs.update(start_event=kernel_events[0].handle, stop_event=kernel_events[1].handle)
        if self.workspace is not None:
            inputs.update(workspace=self.workspace.data_ptr(),
                          workspace_bytes=self.workspace.numel() * 4)
        self.lib.process(self.embed_table_ptrs.data_ptr(), output.data_ptr(), batch,
                         tile_bytes=tile_bytes, grid_blocks=grid_blocks, xcd_segments=xcd_segments,
                         times=times.data_ptr() if times is not None else 0, stream=stream,
                         output_row_stride=row_stride, **inputs)
        if timing:
            n = len(self.embed_tables)
            if not timing_schedules or timing_schedules > n:
                timing_schedules = n
            # device ticks (s_memtime) summed over the tiles of each schedule
            host_times = times.cpu().to(torch.float64)
            task_times = host_times[:timing_schedules]
            self.last_workgroup_ticks = (float(host_times[n]), float(host_times[n + 1]))
            return output, task_times
        return output

    def forward(self, arg_buffers: torch.Tensor, data_buffer_offsets: torch.Tensor,
                scala_args: torch.Tensor = None, extra_buffers: torch.Tensor = None,
                extra_buffer_offsets: torch.Tensor = None, task_mapping: torch.Tensor = None,
                task_tiles: torch.Tensor = None, task_barriers: torch.Tensor = None,
                output_size: int = 0, timing: bool = False, timing_schedules: int = None,
                tile_bytes: int = 0, grid_blocks: int = 0):
        if arg_buffers.dtype != torch.int32 or data_buffer_offsets.dtype != torch.int64:
            raise TypeError("arg_buffers must be int32 and data_buffer_offsets int64")
        if data_buffer_offsets.numel() != len(self.embed_tables) + 1:
            raise ValueError("data_buffer_offsets must have num_features + 1 entries")
        row_bytes = self.output_units * 4
        if output_size % row_bytes != 0:
            raise ValueError(f"output_size={output_size} is not a whole number of "
                             f"{self.output_units}-column fp32 rows")
        batch = output_size // row_bytes
        return self._launch(batch, timing, timing_schedules, tile_bytes, grid_blocks,
                            arg_buffers=arg_buffers.data_ptr(),
                            arg_buffer_offsets=data_buffer_offsets.data_ptr())

    def bind_inputs(self, indices: Sequence[torch.Tensor], offsets: Sequence[torch.Tensor]) -> "BoundInputs":
        """Validate per-feature index / offset tensors once and upload their addresses.  The
        result can be passed to ``forward_indices`` any number of times (the tensors may be
        refilled in place between calls); a call with it costs no per-feature host work, which
        for a model of a thousand features is 0.15 ms per call otherwise."""
        n = len(self.embed_tables)
        if len(indices) != n or len(offsets) != n:
            raise ValueError(f"expected {n} index and offset tensors")
        batch = offsets[0].numel() - 1
        for f in range(n):
            for name, t in (("indices", indices[f]), ("offsets", offsets[f])):
                if t.dtype != torch.int32 or not t.is_contiguous() or t.device.type != "cuda":
                    raise TypeError(f"{name}[{f}] must be a contiguous int32 device tensor")
            if offsets[f].numel() != batch + 1:
                raise ValueError("all features must share one batch size")
        flat = [0] * (2 * n)
        flat[0::2] = [t.data_ptr() for t in indices]
        flat[1::2] = [t.data_ptr() for t in offsets]
        io_ptrs = torch.tensor(flat, dtype=torch.int64, device=self.device)
        # the lengths of the index arrays: a hint that spares the kernel's binding one scattered
        # read per feature (recom_process_args.d_lookup_counts; wrong figures -- tensors refilled
        # with fewer lookups than they hold -- cost balance only)
        counts = torch.tensor([t.numel() for t in indices], dtype=torch.int32, device=self.device)
        return BoundInputs(batch, io_ptrs, (list(indices), list(offsets)), counts)

    def check_inputs(self, indices: Sequence[torch.Tensor], offsets: Sequence[torch.Tensor]) -> None:
        """Debugging aid: raise ``ValueError`` if a launch on these inputs would read outside a
        table or an index array -- offsets that do not start at 0, decrease, or end beyond the
        index array; an index below 0 or beyond its table's rows.  The kernel itself checks
        nothing (neither does the reference's), and an access outside device memory ends the
        process.  Reads the inputs back with stock torch reductions and synchronises, so it is
        meant for tests and for new data pipelines, not for the serving loop."""
        self.bind_inputs(indices, offsets)              # types, shapes, devices
        for f, (idx, off) in enumerate(zip(indices, offsets)):
            rows = self.embed_tables[f].shape[0]
            o = off.to(torch.int64)
            if int(o[0]) != 0:
                raise ValueError(f"feature {f}: offsets[0] = {int(o[0])}, expected 0")
            if o.numel() > 1 and bool((o[1:] < o[:-1]).any()):
                raise ValueError(f"feature {f}: offsets decrease")
            used = int(o[-1])
            if used > idx.numel():
                raise ValueError(f"feature {f}: offsets end at {used}, beyond the {idx.numel()} indices")
            if used > 0:
                lo, hi = int(idx[:used].min()), int(idx[:used].max())
                if lo < 0 or hi >= rows:
                    raise ValueError(f"feature {f}: indices span [{lo}, {hi}], table has {rows} rows")

    def forward_indices(self, indices: Union["BoundInputs", Sequence[torch.Tensor]],
                        offsets: Sequence[torch.Tensor] = None,
                        timing: bool = False, timing_schedules: int = None, tile_bytes: int = 0,
                        grid_blocks: int = 0, schedule_choice: torch.Tensor = None,
                        out: torch.Tensor = None, xcd_segments: int = 0, kernel_events=None):
        """Per-feature int32 device tensors ``indices[f]`` (``[L_f]``) and ``offsets[f]``
        (``[batch + 1]``, exclusive prefix sums, ``offsets[f][0] == 0``) -> ``[batch, sum(dim)]``
        fp32 (with ``timing=True``: ``(output, task_times)``).  ``out``: write into this
        preallocated tensor instead of allocating one.  Instead of the two lists, the result of
        ``bind_inputs`` may be given.  ``kernel_events``: a pair of ``hip_helper.HipEvent`` that
        receives the begin and end of the fused kernel's own dispatch."""
        if isinstance(indices, BoundInputs):
            bound = indices
        else:
            n = len(self.embed_tables)
            if offsets is None or len(indices) != n or len(offsets) != n:
                raise ValueError(f"expected {n} index and offset tensors")
            key = tuple(t.data_ptr() for t in indices) + tuple(t.data_ptr() for t in offsets) \
                + (offsets[0].numel(),)
            if key != self._io_cache_key:
                # new input tensors: validate them and upload their addresses
                self._io_bound = self.bind_inputs(indices, offsets)
                self._io_cache_key = key
            bound = self._io_bound
        batch = bound.batch
        res = self._launch(batch, timing, timing_schedules, tile_bytes, grid_blocks,
                           schedule_choice=schedule_choice, out=out, xcd_segments=xcd_segments,
                           kernel_events=kernel_events, io_ptrs=bound.io_ptrs.data_ptr(),
                           lookup_counts=(bound.lookup_counts.data_ptr()
                                          if bound.lookup_counts is not None else 0))
        if timing:
            return res[0].view(batch, self.output_units), res[1]
        return res.view(batch, self.output_units)


class BoundInputs(NamedTuple):
    """Input tensors of ``FeatEmbed.forward_indices`` with their device address table."""
    batch: int
    io_ptrs: torch.Tensor       # int64 [2 * F] on the device: indices_f, offsets_f addresses
    tensors: tuple              # keeps the bound tensors alive
    lookup_counts: Optional[torch.Tensor] = None    # int32 [F] on the device: len(indices_f)


class FeatProcessEmbed(nn.Module):
    def __init__(self, recom_host, device: torch.device, embed_tables: List[torch.Tensor] = None,
                 table_shapes: List[Tuple[int, int]] = None, librecom_path: str = None,
                 librecom: Union[None, str, RecomLib] = None):
        super(FeatProcessEmbed, self).__init__()
        self.device = device

        if librecom_path:
            librecom = load_library(librecom_path)

        self.embed_layer = FeatEmbed(device=self.device, embed_tables=embed_tables,
                                     table_shapes=table_shapes, librecom=librecom)
        self.preprocess_layer = FeatPreprocess(recom_host, device=self.embed_layer.device,
                                               output_units=self.embed_layer.output_units)
        self.max_concurrent_blocks = self.embed_layer.max_concurrent_blocks

    def forward(self, raw_data: List[List[str]], timing: bool = False, timing_schedules: int = None,
                timing_kernel: bool = False):
        preprocess_result = self.preprocess_layer(raw_data, self.max_concurrent_blocks)
        if not timing_kernel:
            return self.embed_layer(*preprocess_result, timing=timing, timing_schedules=timing_schedules)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        result = self.embed_layer(*preprocess_result, timing=timing, timing_schedules=timing_schedules)
        end.record()
        end.synchronize()
        return result, start.elapsed_time(end)


class RecomModel(nn.Module):
    """Fused embedding followed by an MLP (ReLU between layers, sigmoid at the end), as
    ``RecFlex/rec_modules.py:143-179``."""

    def __init__(self, mlp_unit_nums: List[int], device: torch.device, embed_tables: List[torch.Tensor] = None,
                 table_shapes: List[Tuple[int, int]] = None, librecom: Union[None, str, RecomLib] = None):
        super(RecomModel, self).__init__()
        self.device = device
        self.embed_layer = FeatEmbed(device=self.device, embed_tables=embed_tables,
                                     table_shapes=table_shapes, librecom=librecom)

        layers = nn.ModuleList()
        unit_nums = [self.embed_layer.output_units] + list(mlp_unit_nums) + [1]
        for i in range(len(unit_nums) - 1):
            layers.append(nn.Linear(unit_nums[i], unit_nums[i + 1], bias=True, device=self.embed_layer.device))
            layers.append(nn.Sigmoid() if i + 2 == len(unit_nums) else nn.ReLU())
        self.mlp = nn.Sequential(*layers)

    def forward(self, arg_buffers: torch.Tensor, data_buffer_offsets: torch.Tensor,
                scala_args: torch.Tensor, extra_buffers: torch.Tensor, extra_buffer_offsets: torch.Tensor,
                task_mapping: torch.Tensor, task_tiles: torch.Tensor, task_barriers: torch.Tensor,
                embed_output_size: int):
        embed_output: torch.Tensor = self.embed_layer(
            arg_buffers, data_buffer_offsets, scala_args, extra_buffers, extra_buffer_offsets,
            task_mapping, task_tiles, task_barriers, embed_output_size)
        embed_output = torch.reshape(embed_output, [-1, self.embed_layer.output_units])
        return self.mlp(embed_output)
