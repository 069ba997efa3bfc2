"""Runtime side of the drop-in: the forward-pre-hook that decodes a compressed
block on the fly, the loader that wires DF11 safetensors into a model, and the
compressor that writes them.  Names, signatures, module attribute names and the
on-disk layout follow the reference (dfloat11/dfloat11.py); the decode itself is
the gfx950 kernel behind the C-ABI of include/df11.h, launched on torch's
current stream.

What differs from the reference, by design:
  * the kernel is launched on the caller's (torch's current) stream, not on an
    implicit default stream (reference: dfloat11.py:142-151);
  * each compressed module keeps a small decode workspace on its device (derived
    tables and 512-byte-granular output positions, about 0.2 % of the compressed
    size), built the first time the module runs there;
  * offloaded streams are fetched on a side stream one block ahead of use (the
    reference copies them inside the hook, on the compute stream:
    dfloat11.py:122-128);
  * the correctness check of compress_model decodes on the GPU the module is
    destined for, not on a hard-coded cuda:0 (dfloat11.py:561).
"""
import json
import os
import re
import weakref
from sys import stderr
from typing import Dict, Optional, Union

import torch
import torch.nn as nn

from . import decode as _decode
from .dfloat11_utils import encode_weights, get_32bit_codec, get_codec, get_luts

# Format constants (reference: dfloat11.py:43-49)
version = '0.5.0'
bytes_per_thread = 8
threads_per_block = (512, )
offloaded_tensor_names = ('encoded_exponent', 'sign_mantissa')


class TensorManager:
    """One grow-only BF16 scratch tensor per device, handed out as [:n] slices
    (reference: dfloat11.py:52-100).  All compressed modules of a device decode
    into it, one after the other; stream order is the only guard."""
    _tensors = {}   # device -> tensor

    @staticmethod
    def allocate_bfloat16(device, n_elements):
        if isinstance(device, str):
            device = torch.device(device)
        existing = TensorManager._tensors.get(device)
        if existing is not None:
            if existing.numel() >= n_elements:
                return existing[:n_elements]
            del TensorManager._tensors[device]
            del existing
            torch.cuda.empty_cache()
        new_tensor = torch.empty(n_elements, dtype=torch.bfloat16, device=device)
        print(f'Allocated {n_elements} bf16 on device {device}', file=stderr)
        TensorManager._tensors[device] = new_tensor
        return new_tensor

    @staticmethod
    def clear():
        TensorManager._tensors.clear()


class _OffloadPrefetcher:
    """Copies the offloaded streams of the NEXT compressed module to the device on
    a side stream while the current one decodes and runs.  Which module follows
    which is learnt from the order in which their hooks fire; two device staging
    slots per tensor name alternate, and events order copy -> decode -> slot reuse.

    Modules are referenced weakly: a model that is deleted takes its pinned host
    streams with it, and when the last offloaded module seen on a device is gone
    the device's staging slots and side stream are released too."""

    def __init__(self):
        self.successor = weakref.WeakKeyDictionary()   # module -> weakref of the module that ran after it
        self.pending = weakref.WeakKeyDictionary()     # module -> (dict name -> device tensor, copy-done event, parity)
        self.seen = weakref.WeakKeyDictionary()        # module -> device it was registered for
        self.last = {}           # device -> (weakref of the module whose hook fired last, its parity)
        self.live = {}           # device -> number of living modules registered for it
        self.streams = {}        # device -> side stream
        self.slots = {}          # (device, parity, name) -> device tensor
        self.slot_free = {}      # (device, parity) -> event recorded after the last decode that read the slot
        self.slot_owner = {}     # (device, parity) -> weakref of the module whose streams the slot holds or is receiving
        self.finalizers = weakref.WeakKeyDictionary()  # module -> the finalizer that reports its death
        self.generation = getattr(self, 'generation', 0) + 1   # finalizers of an earlier reset() are void
        self.enabled = True

    # -- the three places that touch the GPU, kept apart so that the bookkeeping can be tested without one
    def _side_stream(self, device):
        side = self.streams.get(device)
        if side is None:
            side = self.streams[device] = torch.cuda.Stream(device=device)
        return side

    def _copy_to_slots(self, module, device, parity):
        side = self._side_stream(device)
        free = self.slot_free.get((device, parity))
        with torch.cuda.stream(side):
            if free is not None:
                side.wait_event(free)          # the decode that last read this slot is done
            tensors = {}
            for name, host in module.offloaded_tensors.items():
                dst = self._slot(device, parity, name, host)
                dst.copy_(host, non_blocking=True)
                tensors[name] = dst
            done = torch.cuda.Event()
            done.record(side)
        return tensors, done

    def _wait_and_mark(self, device, tensors, done):
        current = torch.cuda.current_stream(device)
        current.wait_event(done)
        for t in tensors.values():
            t.record_stream(current)          # allocated on the side stream, read on this one

    def _decode_done_event(self, device):
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(device))
        return ev

    # -- bookkeeping
    def _slot(self, device, parity, name, like):
        key = (device, parity, name)
        buf = self.slots.get(key)
        if buf is None or buf.numel() < like.numel():
            buf = torch.empty(like.numel(), dtype=like.dtype, device=device)
            self.slots[key] = buf
        return buf[:like.numel()]

    def _register(self, module, device):
        if self.seen.get(module) == device:
            return
        if module in self.seen:                # moved to another device: counted there from now on
            self.finalizers.pop(module).detach()
            self._released(self.seen[module], self.generation)
        self.seen[module] = device
        self.live[device] = self.live.get(device, 0) + 1
        self.finalizers[module] = weakref.finalize(module, self._released, device, self.generation)

    def _released(self, device, generation):
        """A module registered for `device` is gone (or has moved away)."""
        if generation != self.generation:
            return
        left = self.live.get(device, 0) - 1
        if left > 0:
            self.live[device] = left
            return
        self.live.pop(device, None)
        self.streams.pop(device, None)
        self.last.pop(device, None)
        for table in (self.slots, self.slot_free, self.slot_owner):
            for key in [k for k in table if k[0] == device]:
                del table[key]

    def _issue(self, module, device, parity):
        """Start the host-to-device copies of `module`'s offloaded tensors on the side stream."""
        tensors, done = self._copy_to_slots(module, device, parity)
        self.pending[module] = (tensors, done, parity)
        self.slot_owner[(device, parity)] = weakref.ref(module)

    def _prefetched(self, module, device):
        """True while the copies issued for `module` are still what its slot holds.
        When modules run in another order than the one learnt (a block skipped, a
        new one in between), a slot can be handed to another module before the
        one it was filled for ever runs."""
        entry = self.pending.get(module)
        if entry is None:
            return False
        owner = self.slot_owner.get((device, entry[2]))
        if owner is None or owner() is not module:
            del self.pending[module]
            return False
        return True

    def fetch(self, module, device):
        """Device copies of `module`'s offloaded tensors, ready on the current stream."""
        self._register(module, device)
        last = self.last.get(device)
        if last is not None:
            before = last[0]()
            if before is not None and before is not module:
                self.successor[before] = weakref.ref(module)
        if not self._prefetched(module, device):
            # first pass, or the prediction missed: the slot the previous module is not using
            self._issue(module, device, (last[1] ^ 1) if last is not None else 0)
        tensors, done, parity = self.pending.pop(module)
        self._wait_and_mark(device, tensors, done)
        self.last[device] = (weakref.ref(module), parity)
        return tensors, parity

    def after_decode(self, module, device, parity):
        """Called once the decode of `module` is enqueued: frees its slot for reuse and
        prefetches the module expected to run next into the other slot."""
        self.slot_free[(device, parity)] = self._decode_done_event(device)
        nxt = self.successor.get(module)
        nxt = nxt() if nxt is not None else None
        if self.enabled and nxt is not None and getattr(nxt, 'offloaded_tensors', None) \
                and not self._prefetched(nxt, device):
            self._issue(nxt, device, parity ^ 1)

    def reset(self):
        self.__init__()


_prefetcher = _OffloadPrefetcher()


_STREAM_NAMES = ('luts', 'encoded_exponent', 'sign_mantissa', 'output_positions', 'gaps')


def _stream_state(module):
    """The five stream tensors of a module as (object, in-place version, address, size)
    entries: what the cached launch arguments and the decode workspace were derived
    from.  A tensor that was replaced shows as another object, one written in place
    (load_state_dict copies into the existing buffers) as another version, and one
    whose storage was rebound (`t.data = other`, `t.set_(...)`: same object, same
    version) as another address or size."""
    state = []
    for name in _STREAM_NAMES:
        t = module._buffers.get(name)
        if t is None and name in getattr(module, 'offloaded_tensors', {}):
            t = module.offloaded_tensors[name]
        state.append((t, t._version, t.data_ptr(), t.numel()) if t is not None else (None, -1, 0, 0))
    return tuple(state)


def _same_streams(module, state):
    """Does _stream_state(module) still equal `state`?  Runs before every cached launch,
    so it builds nothing and leaves at the first difference."""
    buffers = module._buffers
    for name, (was, version, address, numel) in zip(_STREAM_NAMES, state):
        t = buffers.get(name)
        if t is None:
            offloaded = module.__dict__.get('offloaded_tensors')
            t = offloaded.get(name) if offloaded else None
        if t is not was:
            return False
        if t is not None and (t._version != version or t.data_ptr() != address or t.numel() != numel):
            return False
    return True


def _views_in_place(injected):
    """Is every injected `weight` view still the attribute of its module?"""
    for owner, view in injected:
        if owner.__dict__.get('weight') is not view:
            return False
    return True


def _workspace_for(module, device, encoded_exponent, n_elements):
    """The module's decode workspace on `device`: built on first use there, and again
    when any of the stream tensors it was derived from has been replaced or rewritten."""
    cached = module.__dict__.get('_df11_workspace_state')
    ws = getattr(module, '_df11_workspace', None)
    if ws is None or ws.device != device or cached is None or not _same_streams(module, cached):
        # check the layout before anything is launched on it
        sign_mantissa = module.offloaded_tensors['sign_mantissa'] \
            if 'sign_mantissa' in getattr(module, 'offloaded_tensors', {}) else module.sign_mantissa
        _decode.validate_stream(module.luts, encoded_exponent, sign_mantissa, module.output_positions,
                                module.gaps, type(module).__name__)
        ws, max_sub = _decode.prepare(module.luts, encoded_exponent, module.output_positions,
                                      module.gaps, n_elements)
        # plain attributes, not buffers: derived data must not leak into state_dict()
        object.__setattr__(module, '_df11_workspace', ws)
        object.__setattr__(module, '_df11_max_sub', max_sub)
        object.__setattr__(module, '_df11_workspace_state', _stream_state(module))
    return module._df11_workspace, module._df11_max_sub


# An embedding's forward reads the rows it looks up and nothing else, so its hook decodes
# only those (df11_decode_rows) once the module's launch arguments are bound, i.e. from
# its second call on; set to False to decode the whole table before every lookup, as the
# reference does (reference: dfloat11.py:153-157).
EMBEDDING_ROW_DECODE = True


def _looked_up_rows(module, inputs, device):
    """The row numbers an nn.Embedding is about to look up, as a contiguous int64 tensor on
    `device`, if decoding just those rows is the cheaper call; else None."""
    if not EMBEDDING_ROW_DECODE or not inputs or not isinstance(inputs[0], torch.Tensor):
        return None
    ids = inputs[0]
    if ids.dtype != torch.int64 or ids.device != device or ids.numel() == 0 \
            or ids.numel() * 4 > module.num_embeddings:
        return None
    return ids if ids.is_contiguous() else ids.contiguous()


def get_hook(threads_per_block, bytes_per_thread):
    """Forward-pre-hook factory (reference: dfloat11.py:103-176).  The hook reads
    the module attributes luts, encoded_exponent, sign_mantissa, output_positions,
    gaps, split_positions, weight_injection_modules, offloaded_tensors, decodes into
    the device's shared BF16 buffer and installs `weight` views of it."""
    threads_per_block = tuple(threads_per_block)
    if threads_per_block != (512, ) or bytes_per_thread != 8:
        raise NotImplementedError(
            f'DF11 streams with threads_per_block={threads_per_block}, bytes_per_thread={bytes_per_thread} '
            'are not supported (only 512 x 8)')

    def decode_hook(module, inputs):
        device = module.luts.device
        if device.type != 'cuda':
            raise RuntimeError(
                f'DFloat11 module is on {device}: weights are decoded on the GPU only; move the model to a GPU')

        # Resident streams: the launch arguments and the injected weight views stay
        # valid while the stream tensors and the device's shared buffer are the very
        # same objects and nobody has put another `weight` in place of a view, so
        # later calls are one library call and nothing else.
        plan = module.__dict__.get('_df11_plan')
        if plan is not None and plan[0] is TensorManager._tensors.get(device) \
                and _same_streams(module, plan[1]) and _views_in_place(plan[3]):
            row_ids = _looked_up_rows(module, inputs, device) if plan[4] else None
            if row_ids is None or not _decode.launch_rows(plan[2], device, row_ids, plan[4]):
                _decode.launch(plan[2], device)
            return

        # Each of the two large streams comes from the prefetcher when the module holds it in
        # host memory, else from the module's own buffer (a module may have only one of them
        # offloaded: reference dfloat11.py:123-128 moves whatever offloaded_tensors holds).
        parity = None
        fetched = {}
        if getattr(module, 'offloaded_tensors', None):
            fetched, parity = _prefetcher.fetch(module, device)
        encoded_exponent = fetched['encoded_exponent'] if 'encoded_exponent' in fetched else module.encoded_exponent
        sign_mantissa = fetched['sign_mantissa'] if 'sign_mantissa' in fetched else module.sign_mantissa

        n_elements = sign_mantissa.numel()
        reconstructed = TensorManager.allocate_bfloat16(device, n_elements)
        workspace, max_sub = _workspace_for(module, device, encoded_exponent, n_elements)
        bound = _decode.bind(module.luts, encoded_exponent, sign_mantissa, module.output_positions,
                             module.gaps, reconstructed, workspace, max_sub)
        _decode.launch(bound, device)

        if isinstance(module, nn.Linear):
            module.weight = reconstructed.view(module.out_features, module.in_features)
            injected = [(module, module.weight)]
        elif isinstance(module, nn.Embedding):
            module.weight = reconstructed.view(module.num_embeddings, module.embedding_dim)
            injected = [(module, module.weight)]
        else:
            injected = []
            weights = torch.tensor_split(reconstructed, module.split_positions)
            for sub_module, weight in zip(module.weight_injection_modules, weights):
                sub_module.weight = weight.view(sub_module.out_features, sub_module.in_features)
                injected.append((sub_module, sub_module.weight))

        if parity is not None:
            _prefetcher.after_decode(module, device, parity)
        else:
            row_elements = module.embedding_dim if isinstance(module, nn.Embedding) else 0
            object.__setattr__(module, '_df11_plan', (TensorManager._tensors.get(device), _stream_state(module),
                                                      bound, injected, row_elements))

    return decode_hook


def _module_at(model, parts):
    module = model
    for part in parts:
        if not hasattr(module, part):
            return None
        module = getattr(module, part)
    return module


def _drop_weight(module):
    if 'weight' in module._parameters or hasattr(module, 'weight'):
        tmp = module.weight
        delattr(module, 'weight')
        del tmp


def load_and_replace_tensors(
    model,
    directory_path,
    dfloat11_config,
    cpu_offload=False,
    cpu_offload_blocks=None,
    pin_memory=True,
    from_single_file=False,
):
    """Reads DF11 safetensors and prepares `model` for on-the-fly decompression
    (reference: dfloat11.py:179-308): plain tensors are copied into their
    parameters/buffers; the DF11 components become buffers (or pinned host tensors
    when offloaded) of the module they belong to, which gets the decode hook and
    loses its `weight` attributes."""
    from safetensors.torch import load_file
    from tqdm import tqdm

    threads = dfloat11_config['threads_per_block']
    bpt = dfloat11_config['bytes_per_thread']
    pattern_dict = dfloat11_config['pattern_dict']

    files = [directory_path] if from_single_file else sorted(
        os.path.join(directory_path, f) for f in os.listdir(directory_path) if f.endswith('.safetensors'))
    desc = 'Loading DFloat11 safetensors'
    if cpu_offload:
        desc += ' (offloaded to CPU' + (', memory pinned' if pin_memory else '') + ')'

    params = dict(model.named_parameters())
    buffers = dict(model.named_buffers())

    for file_path in tqdm(files, desc=desc):
        for tensor_name, tensor_value in load_file(file_path).items():
            target = params.get(tensor_name)
            if target is None:
                target = buffers.get(tensor_name)
            if target is not None:
                if target.shape == tensor_value.shape:
                    target.data.copy_(tensor_value)
                else:
                    print(f'Shape mismatch for {tensor_name}: model {target.shape} vs loaded {tensor_value.shape}',
                          file=stderr)
                continue

            parts = tensor_name.split('.')
            module = _module_at(model, parts[:-1])
            if module is None:
                print(f'Cannot find module path for {tensor_name}', file=stderr)
                continue
            leaf = parts[-1]

            if leaf == 'split_positions':
                setattr(module, 'split_positions', tensor_value.tolist())
                continue

            offload = (cpu_offload and (cpu_offload_blocks is None or cpu_offload_blocks > 0)
                       and leaf in offloaded_tensor_names)
            if offload:
                if not hasattr(module, 'offloaded_tensors'):
                    setattr(module, 'offloaded_tensors', {})
                module.offloaded_tensors[leaf] = tensor_value.pin_memory() if pin_memory else tensor_value
                if (cpu_offload_blocks is not None and cpu_offload_blocks > 0
                        and len(module.offloaded_tensors) == len(offloaded_tensor_names)):
                    cpu_offload_blocks -= 1
            else:
                module.register_buffer(leaf, tensor_value)

            if leaf == 'encoded_exponent':
                module.register_forward_pre_hook(get_hook(threads, bpt))
                module_name = '.'.join(parts[:-1])
                for pattern, attr_names in pattern_dict.items():
                    if not re.fullmatch(pattern, module_name):
                        continue
                    if isinstance(module, (nn.Embedding, nn.Linear)):
                        _drop_weight(module)
                    else:
                        module.weight_injection_modules = []
                        for attr_path in attr_names:
                            sub = _module_at(module, attr_path.split('.'))
                            if sub is None:
                                raise AttributeError(f'{module_name} has no sub-module {attr_path}')
                            _drop_weight(sub)
                            module.weight_injection_modules.append(sub)
            elif leaf == 'output_positions':
                # kept for parity with the reference's attribute set (dfloat11.py:299-306):
                # 512 * 4 + 4 + 2 * max(elements per 4096-byte block)
                pos = tensor_value.view(torch.uint8).view(torch.int32).to(torch.int64) & 0xFFFFFFFF
                widest = int((pos[1:] - pos[:-1]).max().item()) if pos.numel() > 1 else 0
                setattr(module, 'shared_mem_size', threads[0] * 4 + 4 + widest * 2)

    return model


def get_no_split_classes(model, pattern_dict):
    """Class names of the compressed blocks: they must stay on one device together
    with their decode buffers (reference: dfloat11.py:311-333)."""
    names = []
    for pattern in pattern_dict:
        for full_name, sub_module in model.named_modules():
            if re.fullmatch(pattern, full_name) and sub_module.__class__.__name__ not in names:
                names.append(sub_module.__class__.__name__)
    return names


class DFloat11Model:
    """Loads models whose weights are stored in DF11 (reference: dfloat11.py:336-493)."""

    @classmethod
    def from_pretrained(
        cls,
        dfloat11_model_name_or_path: str,
        device: Optional[str] = None,
        device_map: str = 'auto',
        max_memory: Optional[Dict[Union[int, str], Union[int, str]]] = None,
        bfloat16_model=None,
        cpu_offload: bool = False,
        cpu_offload_blocks: Optional[int] = None,
        pin_memory: bool = True,
        from_single_file: bool = False,
        pattern_dict: Optional[Dict[str, list]] = None,
        **kwargs,
    ):
        if from_single_file:
            if os.path.isfile(dfloat11_model_name_or_path):
                path = dfloat11_model_name_or_path
            elif os.path.isdir(dfloat11_model_name_or_path):
                raise IsADirectoryError(
                    'Expected `dfloat11_model_name_or_path` to be the path to a safetensors file, '
                    f'but found a directory: "{dfloat11_model_name_or_path}".')
            else:
                raise FileNotFoundError(f'The file "{dfloat11_model_name_or_path}" does not exist.')
        elif os.path.exists(dfloat11_model_name_or_path):
            path = dfloat11_model_name_or_path
        else:
            path = dfloat11_model_name_or_path.replace('/', '__')
            if not os.path.exists(path):
                from huggingface_hub import snapshot_download
                snapshot_download(dfloat11_model_name_or_path, local_dir=path)

        if bfloat16_model:
            if from_single_file:
                config = {'dfloat11_config': {
                    'version': version,
                    'threads_per_block': threads_per_block,
                    'bytes_per_thread': bytes_per_thread,
                    'pattern_dict': pattern_dict,
                }}
            else:
                with open(os.path.join(path, 'config.json'), 'r', encoding='utf-8') as f:
                    config = json.load(f)
            model = bfloat16_model
        else:
            from transformers import AutoConfig, AutoModelForCausalLM, GenerationConfig
            try:                                    # moved between transformers releases
                from transformers.modeling_utils import no_init_weights
            except ImportError:
                from transformers.initialization import no_init_weights
            config = AutoConfig.from_pretrained(path)
            with no_init_weights():
                model = AutoModelForCausalLM.from_config(config, torch_dtype=torch.bfloat16, **kwargs)
                model.tie_weights()
                model.eval()
            try:
                model.generation_config = GenerationConfig.from_pretrained(path)
            except Exception:
                pass

        if isinstance(config, dict) and 'dfloat11_config' in config:
            dfloat11_config = config['dfloat11_config']
        elif hasattr(config, 'dfloat11_config'):
            dfloat11_config = config.dfloat11_config
        else:
            raise AttributeError(
                '"dfloat11_config" not found: it is expected to be found in the config file or passed as an argument.')

        load_and_replace_tensors(
            model, path, dfloat11_config,
            cpu_offload=cpu_offload, cpu_offload_blocks=cpu_offload_blocks,
            pin_memory=pin_memory, from_single_file=from_single_file,
        )

        if not cpu_offload:
            model_bytes = sum(t.nbytes for t in model.state_dict().values())
            print(f'Total model size: {model_bytes / 1e9:0.4f} GB', file=stderr)

        if device:
            model = model.to(device)
        else:
            assert device_map == 'auto', "device_map should be 'auto' if no specific device is provided."
            from accelerate import dispatch_model, infer_auto_device_map
            from accelerate.utils import get_balanced_memory
            no_split = get_no_split_classes(model, dfloat11_config['pattern_dict'])
            max_memory = get_balanced_memory(model, max_memory=max_memory, no_split_module_classes=no_split)
            dmap = infer_auto_device_map(model, max_memory=max_memory, no_split_module_classes=no_split)
            model = dispatch_model(model, dmap)
            if any(p.device.type == 'cpu' for p in model.parameters()):
                print('Warning: Some model layers are on CPU. For inference, ensure the model is fully loaded '
                      'onto GPUs.', file=stderr)
        return model

    @classmethod
    def from_single_file(
        cls,
        dfloat11_model_path: str,
        pattern_dict: Dict[str, list],
        bfloat16_model,
        device: Optional[str] = None,
        device_map: str = 'auto',
        max_memory: Optional[Dict[Union[int, str], Union[int, str]]] = None,
        cpu_offload: bool = False,
        cpu_offload_blocks: Optional[int] = None,
        pin_memory: bool = True,
    ):
        return cls.from_pretrained(
            dfloat11_model_name_or_path=dfloat11_model_path, device=device, device_map=device_map,
            max_memory=max_memory, bfloat16_model=bfloat16_model, cpu_offload=cpu_offload,
            cpu_offload_blocks=cpu_offload_blocks, pin_memory=pin_memory, from_single_file=True,
            pattern_dict=pattern_dict,
        )


def _check_on_gpu(full_name, weights, luts, encoded, other_8bits, output_positions, gaps, device):
    """decode(encode(W)) == W on the GPU (reference: dfloat11.py:560-591)."""
    if not torch.cuda.is_available():
        raise RuntimeError('check_correctness=True needs a GPU: DF11 streams are decoded on the GPU only')
    dev = torch.device(device if device is not None else f'cuda:{torch.cuda.current_device()}')
    d_luts, d_enc, d_sm, d_gaps = (t.to(dev) for t in (luts, encoded, other_8bits, gaps))
    d_pos = output_positions.view(torch.uint8).to(dev)
    out = torch.empty(other_8bits.numel(), dtype=torch.bfloat16, device=dev)
    ws, max_sub = _decode.prepare(d_luts, d_enc, d_pos, d_gaps, other_8bits.numel())
    _decode.decode(d_luts, d_enc, d_sm, d_pos, d_gaps, out, ws, max_sub)
    original = torch.cat(weights).view(torch.int16)
    if not torch.equal(original, out.cpu().view(torch.int16)):
        raise RuntimeError(
            'Correctness check failed: the decompressed weights do not match the original weights for '
            f'module "{full_name}".')
    print('Correctness check passed: decompressed weights match the original weights.')


def compress_model(
    model,
    pattern_dict: Dict[str, list],
    save_path: str,
    block_range: list = [0, 10000],
    save_single_file: bool = True,
    check_correctness: bool = True,
    check_device: Optional[str] = None,
):
    """Compresses the BF16 weights selected by `pattern_dict` and saves the model
    (reference: dfloat11.py:496-636): one DF11 stream per matched module, its
    sub-module weights concatenated in the order listed."""
    from safetensors.torch import save_file

    os.makedirs(save_path, exist_ok=True)
    block_index = 0
    save_model = True
    for pattern, attr_names in pattern_dict.items():
        if not save_model:
            break
        for full_name, sub_module in list(model.named_modules()):
            if not re.fullmatch(pattern, full_name):
                continue
            if not save_single_file:
                # each block goes to its own file; detach it from the tree that is saved last
                if '.' in full_name:
                    parent_name, child_name = full_name.rsplit('.', 1)
                    setattr(model.get_submodule(parent_name), child_name, None)
                else:
                    setattr(model, full_name, None)

            block_index += 1
            if block_index <= block_range[0]:
                continue
            if block_index > block_range[1]:
                save_model = False
                break

            if isinstance(sub_module, (nn.Embedding, nn.Linear)):
                targets = [(full_name, sub_module)]
            else:
                targets = []
                for attr_path in attr_names:
                    target = _module_at(sub_module, attr_path.split('.'))
                    if target is None:
                        raise AttributeError(f'{full_name} has no sub-module {attr_path}')
                    targets.append((f'{full_name}.{attr_path}', target))
            weights = []
            for name, target in targets:
                assert target.weight.data.dtype == torch.bfloat16, (
                    f"Expected weights to be in bfloat16 format for compression, but '{name}' has dtype "
                    f'{target.weight.data.dtype}')
                weights.append(target.weight.data.detach().cpu().flatten())
                delattr(target, 'weight')

            _, counter = get_codec(torch.cat(weights))
            codec, _, table = get_32bit_codec(counter)
            luts = get_luts(table)
            encoded, other_8bits, output_positions, gaps, split_positions = encode_weights(
                weights, codec, bytes_per_thread, threads_per_block[0])
            ratio = (encoded.numel() + other_8bits.numel() + output_positions.numel() * 4 + gaps.numel()) * 100 \
                / (other_8bits.numel() * 2)
            print(f'{full_name}: compression factor {ratio:.2f}%')

            if check_correctness:
                _check_on_gpu(full_name, weights, luts, encoded, other_8bits, output_positions, gaps, check_device)

            sub_module.register_buffer('luts', luts)
            sub_module.register_buffer('encoded_exponent', encoded)
            sub_module.register_buffer('sign_mantissa', other_8bits)
            sub_module.register_buffer('output_positions', output_positions.view(torch.uint8))
            sub_module.register_buffer('gaps', gaps)
            sub_module.register_buffer('split_positions', split_positions)

            if not save_single_file:
                state = {f'{full_name}.{key}': value for key, value in sub_module.state_dict().items()}
                save_file(state, os.path.join(save_path, full_name.replace('.', '_') + '.safetensors'))

    if save_model:
        dfloat11_config = {
            'version': version,
            'threads_per_block': threads_per_block,
            'bytes_per_thread': bytes_per_thread,
            'pattern_dict': pattern_dict,
        }
        if hasattr(model, 'config'):
            try:
                model.config.dfloat11_config = dfloat11_config
            except Exception:
                pass
        if hasattr(model, 'save_pretrained') and not save_single_file:
            model.save_pretrained(save_path)
        else:
            save_file({k: v.contiguous() for k, v in model.state_dict().items()},
                      os.path.join(save_path, 'model.safetensors'))

        config_path = os.path.join(save_path, 'config.json')
        save_config = True
        if os.path.exists(config_path):
            with open(config_path, 'r', encoding='utf-8') as f:
                existing = json.load(f)
            if isinstance(existing.get('dfloat11_config'), dict):
                save_config = False
        if save_config:
            with open(config_path, 'w') as config_file:
                json.dump({'dfloat11_config': dfloat11_config}, config_file, indent=2)
