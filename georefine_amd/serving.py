"""Modules that keep coded weights resident and decode them inside the matmul.

Same surface as the reference's serving adapters (GCR/bitexact_context_serving.py:346-400,
GCR/bitexact_context_mtp.py:279-295, GCR/bitexact_predictive_serving.py:490-523): a loader
builds one tensor object per coded weight through an injectable factory and wraps it in
``BctxLinear`` / ``BctxEmbedding``; predictive weights resolve their reference tensors at
decode time.  The difference is ``BctxLinear.forward``: where the reference decodes a dense
transient and calls ``F.linear``, this one calls the tensor's fused ``linear`` when it has
one, which is the slot the reference leaves open (GCR/bitexact_context_serving.py:3-5).
"""
from __future__ import annotations

import threading

import torch
from torch import nn


class ContextServingError(RuntimeError):
    """Malformed or incomplete coded-weight module."""


def hip_tensor_factory(frame, *, stride=1024, device="cuda:0", fused_segment=None, residual_block=None):
    """The ``tensor_factory`` to hand to ``load_bctx_model`` (GCR/bitexact_context_serving.py:416,560).
    ``fused_segment`` fixes the segment length of the fused index (matrices that are to share a
    launch need one length); the loader passes it to factories that take it.  ``residual_block``
    (``functools.partial(hip_tensor_factory, residual_block=16)``): the rows per block of the
    resident residual order; 16 suits matrices that are served in batches (the matrix-core
    kernel's waves hold sixteen rows), the default the one-row GEMV."""
    from .bitexact_context_gpu import HipContextTensor
    return HipContextTensor(frame, stride=stride, device=device, fused_segment=fused_segment,
                            residual_block=residual_block)


def hip_predictive_factory(frame, reference_uint16_numpy, stride=1024, device="cuda:0", *, fused_segment=None):
    """The ``predictive_factory`` of ``load_predictive_model`` (GCR/bitexact_predictive_serving.py:918-924).
    ``fused_segment``: the tile walker's segment length, given by the loader to siblings that
    are to share launches (they need one length)."""
    from .bitexact_predictive_gpu import HipPredictiveTensor
    return HipPredictiveTensor(frame, reference_uint16_numpy, stride=stride, device=device, fused_segment=fused_segment)


class SharedProducts:
    """Sibling linears that are applied to the same tensor one after the other (q/k/v
    projections, gate and up) as one launch: the first member called with a tensor runs the
    whole group and keeps the outputs, the others pick theirs up.  Every output is handed out
    once: when the last member has taken its own, or a member asks again, or the tensor differs
    (identity, version counter, address, shape), the next call runs the group anew.  Within
    one pass the kept outputs assume that the activations were not rewritten behind the
    version counter (a kernel writing through a raw pointer, a graph replay): callers that do
    that between the members' calls must not share launches."""

    def __init__(self, group, biases, batch_invariant=False):
        self.group, self.biases, self.batch_invariant = group, list(biases), batch_invariant
        self.launches = 0
        self._key = self._x = self._outs = None
        self._taken = set()

    def output(self, index, x):
        key = (id(x), x._version, x.data_ptr(), tuple(x.shape), tuple(x.stride()))
        if key != self._key or self._outs is None or self._x() is not x or index in self._taken:
            import weakref
            self._outs = list(self.group.linear(x, self.biases, batch_invariant=self.batch_invariant))
            self._key, self._x, self._taken = key, weakref.ref(x), set()
            self.launches += 1
        out, self._outs[index] = self._outs[index], None
        self._taken.add(index)
        if len(self._taken) == len(self._outs):  # the pass is over: nothing is kept beyond it
            self._key = self._x = self._outs = None
            self._taken = set()
        return out


def prepare_metadata(package, cache_dir):
    """Verify the package's metadata sidecars (the model's configuration files) and return a
    directory that holds them, outside the package: the package's own ``sidecars/`` directory when
    it carries one, else ``cache_dir/<SHA-256 of model-assets.tar.xz>/sidecars``, extracted once and
    re-checked file by file when it already exists (GCR/bitexact_context_serving.py:175-274).  A
    builder-written package pins thirteen of them; anything else is refused, as is a cache inside
    the package."""
    import hashlib
    import os
    import shutil
    import tempfile
    from pathlib import Path, PurePosixPath

    from . import bitexact_context_package as pkg
    package, cache_dir = Path(package).resolve(), Path(cache_dir).resolve()
    if cache_dir == package or package in cache_dir.parents:
        raise ContextServingError("metadata cache must be outside the immutable package")
    try:
        manifest, _ = pkg.read_manifest(package)
        members = pkg.read_metadata(package, manifest)
    except pkg.PackageError as exc:
        raise ContextServingError(str(exc)) from exc
    pins = manifest.get("metadata_assets") or {}
    if len(pins) != 13:
        raise ContextServingError("BCTX v1 metadata inventory must contain 13 sidecars")
    if (package / "sidecars").exists():  # checked against the pins by read_metadata
        return package / "sidecars"
    archive_sha = hashlib.sha256((package / "model-assets.tar.xz").read_bytes()).hexdigest()
    cache_dir.mkdir(parents=True, exist_ok=True)
    destination = cache_dir / archive_sha
    if destination.is_symlink():
        raise ContextServingError("metadata cache destination must not be a symlink")
    if destination.exists():
        if not destination.is_dir():
            raise ContextServingError("metadata cache destination is not a directory")
        present = {}
        for path in destination.rglob("*"):
            if path.is_symlink():
                raise ContextServingError("metadata cache contains a symlink")
            if path.is_file():
                present[path.relative_to(destination).as_posix()] = path
        if set(present) != set(pins):
            raise ContextServingError("existing metadata cache inventory mismatch")
        for name, pin in pins.items():
            payload = present[name].read_bytes()
            if len(payload) != pin["bytes"] or hashlib.sha256(payload).hexdigest() != pin["sha256"]:
                raise ContextServingError(f"existing metadata cache integrity mismatch: {name}")
    else:
        staging = Path(tempfile.mkdtemp(prefix=archive_sha + ".partial-", dir=cache_dir))
        try:
            for name, payload in members.items():
                target = staging.joinpath(*PurePosixPath(name).parts)
                target.parent.mkdir(parents=True, exist_ok=True)
                target.write_bytes(payload)
            os.replace(staging, destination)
        except Exception:
            shutil.rmtree(staging, ignore_errors=True)
            raise
    return destination / "sidecars"


def decode_errors(model):
    """Names of the coded modules of ``model`` whose device error word is set (a segment did
    not end on its checkpoint in some launch since the word was last cleared).  The fused
    kernels never trap and ``linear`` does not read the word back on every call; a server calls
    this between steps, or every so many steps: one small device-to-host read per module."""
    bad = []
    for name, module in model.named_modules():
        weight = getattr(module, "context_weight", None)
        words = [getattr(getattr(weight, "native", weight), "error", None)]
        if getattr(module, "shared", None) is not None:
            words.append(getattr(module.shared[0].group, "error", None))
        if any(w is not None and int(w.item()) != 0 for w in words):
            bad.append(name)
    return bad


class BctxLinear(nn.Module):
    """Linear layer whose weight stays compressed; ``batch_invariant=True`` sends every call
    through the matrix-core kernel so a row never depends on its batch, ``False`` lets the row
    count pick the fastest kernel, ``None`` leaves the choice to the tensor's own policy
    (``HipContextTensor.m_invariant``)."""

    def __init__(self, tensor, bias=None, *, batch_invariant=None):
        super().__init__()
        if len(tensor.shape) != 2:
            raise ContextServingError("linear BCTX weight must be rank two")
        self.context_weight = tensor
        self.out_features, self.in_features = map(int, tensor.shape)
        self.batch_invariant = batch_invariant
        self.forward_calls = 0
        self.weight_materializations = 0
        self.shared = None  # (SharedProducts, index) when siblings share a launch
        self.register_parameter("bias", bias)

    @property
    def weight(self):
        """Dense transient for callers that need the matrix itself; never retained."""
        self.weight_materializations += 1
        return self.context_weight.decode()

    def forward(self, x):
        self.forward_calls += 1
        if self.shared is not None and x.dtype == torch.bfloat16 and x.is_cuda:
            return self.shared[0].output(self.shared[1], x)
        fused = getattr(self.context_weight, "linear", None)
        if fused is not None and x.dtype == torch.bfloat16:
            return fused(x, self.bias, batch_invariant=self.batch_invariant)
        weight = self.weight
        if self.bias is None and x.ndim > 2 and not x.is_contiguous():
            # keep the 2-D matmul dispatch of an ordinary Linear (GCR/bitexact_context_serving.py:369-375)
            out = torch.nn.functional.linear(x.reshape(-1, x.shape[-1]), weight)
            return out.reshape(*x.shape[:-1], self.out_features)
        return torch.nn.functional.linear(x, weight, self.bias)


BCTXLinear = BctxLinear  # name used by the MTP head loader (GCR/bitexact_context_mtp.py:279)


class BctxEmbedding(nn.Module):
    """Embedding table that stays compressed; rows are decoded by indexed gather."""

    def __init__(self, tensor, *, padding_idx=None):
        super().__init__()
        if len(tensor.shape) != 2:
            raise ContextServingError("embedding BCTX weight must be rank two")
        self.context_weight = tensor
        self.num_embeddings, self.embedding_dim = map(int, tensor.shape)
        self.padding_idx = padding_idx
        self.forward_calls = 0
        self.weight_materializations = 0

    @property
    def weight(self):
        self.weight_materializations += 1
        return self.context_weight.decode()

    def forward(self, input):
        self.forward_calls += 1
        return self.context_weight.gather_rows(input)


class PredictiveContextTensor:
    """PPCX weight that resolves its reference tensors when decoded
    (GCR/bitexact_predictive_serving.py:490-523): one reference is used as is, two are mixed
    by ``predictor(up, gate, coefficients)``; ``transform == "target transpose"`` stores the
    frame transposed.

    ``row_major``: a coded tensor of the weight in the model's own orientation, made at load from
    the decoded frame (``reframe`` below); products, decodes and row gathers then go to it and
    the predictive frame's device buffers are released."""

    def __init__(self, native, references, *, predictor=None, coefficients=None, transform=None, shape,
                 source_sha256, frame_sha256, resident_bytes):
        self.native = native
        self.row_major = None
        self.references = tuple(references)
        self.predictor = predictor
        self.coefficients = coefficients
        self.transform = transform
        self.shape = tuple(shape)
        self.source_sha256 = source_sha256
        self.frame_sha256 = frame_sha256
        self.resident_bytes = resident_bytes
        self._decode_lock = threading.RLock()

    def _needs_reference(self):
        """False when the native tensor keeps the contexts of its reference and takes the tile
        walker: nothing of the references is then read after load."""
        return not (getattr(self.native, "has_contexts", False) and getattr(self.native, "fused", None) is not None)

    def reframe(self, tensor_factory, *, stride, device, encoder=None):
        """A frame stored transposed holds W^T row by row: the walk produces words along the
        product's K axis, which no sink of the tile walker can contract.  The reference's shipped
        servers re-frame their Context weights at start-up (GS/predictive_tbe.py:1-15); this does
        the same for such targets, once: the frame is decoded on the device (the index builder has
        already checked it against its digests), turned, encoded row-major with the context
        codec's encoder, and the new frame is indexed like any other -- the decoded words of the
        result must hash to the receipt's ``source_sha256`` of the tensor.  Every later product is
        then one fused launch and ``decode()`` a fused decode; the predictive frame's device
        buffers are released.  Returns the new tensor."""
        import numpy as np
        if encoder is None:
            from .bitexact_context_codec import encode as encoder
        with self._decode_lock:
            words = self.decode(check=True).view(torch.uint16).cpu().numpy()
            tensor = tensor_factory(encoder(np.ascontiguousarray(words)), stride=stride, device=device)
            if tuple(tensor.shape) != tuple(words.shape) or tensor.source_sha256 != self.source_sha256:
                raise ContextServingError("re-framed tensor does not reproduce the decoded source")
            self.row_major = tensor
            self.resident_bytes = int(tensor.resident_bytes)
            self.native = None  # its device buffers go with it
            self.references = ()
        return tensor

    def decode(self, *, check=True):
        if self.row_major is not None:
            return self.row_major.decode(check=check)
        with self._decode_lock:
            value = self.native.decode(self._reference(check) if self._needs_reference() else None, check=check)
            if self.transform == "target transpose":
                value = value.transpose(-2, -1).contiguous()
            return value

    def gather_rows(self, ids, *, check=True):
        if self.row_major is not None:
            return self.row_major.gather_rows(ids, check=check)
        return self.decode(check=check)[ids]

    def _reference(self, check):
        refs = [ctx.decode(check=check) for ctx in self.references]
        if len(refs) == 1:
            return refs[0]
        if self.predictor is None:
            from .bitexact_predictive_mix import predict as default_predictor
            self.predictor = default_predictor
        return self.predictor(refs[0], refs[1], self.coefficients)

    def linear(self, x, bias=None, *, check=False, batch_invariant=None):
        """x W^T + bias.  A frame stored untransposed goes through the native tensor's fused
        product: one launch that decodes and contracts, with the contexts of the reference read
        from the plane kept at load (a native tensor without that plane gets the reference
        decoded first); a transposed frame holds W^T row by row, so it is decoded and multiplied
        densely -- unless it was re-framed at load (``reframe``), in which case the row-major tensor's
        fused product runs."""
        if self.row_major is not None:
            fused = getattr(self.row_major, "linear", None)
            if fused is None:  # a tensor class without a fused product
                return torch.nn.functional.linear(x, self.row_major.decode(check=check), bias)
            return fused(x, bias, check=check, batch_invariant=batch_invariant)
        fused = getattr(self.native, "linear", None)
        if fused is None or self.transform == "target transpose":
            return torch.nn.functional.linear(x, self.decode(check=check), bias)
        with self._decode_lock:
            return fused(self._reference(check) if self._needs_reference() else None, x, bias, check=check,
                         batch_invariant=batch_invariant)


def _launch_group(weights):
    """One grouped launch for sibling weights, or None when they do not all take the same
    walker: tensors of the context codec (a predictive weight re-framed at load counts as its
    row-major tensor) share ``HipLinearGroup``; predictive weights stored untransposed whose
    native tensors keep their context planes share ``HipPredictiveGroup``."""
    from .bitexact_context_gpu import HipContextTensor, HipLinearGroup
    effective = [getattr(w, "row_major", None) or w for w in weights]
    if all(isinstance(w, HipContextTensor) for w in effective):
        return HipLinearGroup(effective)
    from .bitexact_predictive_gpu import HipPredictiveGroup, HipPredictiveTensor
    if all(isinstance(w, PredictiveContextTensor) and w.transform != "target transpose"
           and isinstance(w.native, HipPredictiveTensor) and not w._needs_reference() for w in effective):
        return HipPredictiveGroup([w.native for w in effective])
    return None


# ----------------------------------------------------------------------------- loader

def _parent_and_attr(model, dotted):
    parent_name, _, attr = dotted.rpartition(".")
    return (model.get_submodule(parent_name) if parent_name else model), attr


def _runtime_dtype(model, name, parameter, requested):
    """The requested dtype, except parameters a module pins to fp32 by name pattern
    (``_keep_in_fp32_modules_strict``; GCR/bitexact_context_serving.py:76-89)."""
    from fnmatch import fnmatchcase
    if not parameter.is_floating_point():
        return parameter.dtype
    patterns = []
    for _, module in model.named_modules():
        patterns.extend(str(p) for p in (getattr(module, "_keep_in_fp32_modules_strict", ()) or ()))
        if requested == torch.float16:
            patterns.extend(str(p) for p in (getattr(module, "_keep_in_fp32_modules", ()) or ()))
    return torch.float32 if any(fnmatchcase(name, p) for p in patterns) else requested


def load_bctx_model(package, *, model_factory, device="cuda:0", dtype=torch.bfloat16, stride=1024,
                    tensor_factory=None, predictive_factory=None, mix_predictor=None, host_decoder=None,
                    loader_workers=1, batch_invariant=False, log=print, progress_callback=None,
                    share_launches=(), reframe_transposed=True, check_inventory=None, optional_files=("decoder/",)):
    """Build ``model_factory()`` on the meta device and fill it from a BCTX package without
    ever holding a dense checkpoint: returns ``(model, receipt)``.

    The procedure and its checks are the reference loader's
    (GCR/bitexact_context_serving.py:409-712): every ``nn.Linear`` / ``nn.Embedding`` whose
    weight has a receipt keeps the frame resident on ``device`` behind ``BctxLinear`` /
    ``BctxEmbedding`` (one ``tensor_factory(frame, stride=, device=)`` call each, from
    ``loader_workers`` threads); the object's geometry, decoded-source digest, frame digest
    and ``resident_bytes`` are checked against the receipt.  Every other parameter and every
    linear bias is decoded on the host, digest checked, and installed dense.  The model must
    end with no meta tensor left.

    Weights listed under the manifest's ``selected_candidates`` are PPCX frames coded against
    other tensors of the package (GCR/bitexact_predictive_serving.py:880-935): their
    references get tensor objects first, ``predictive_factory(frame, reference_words,
    stride=, device=)`` indexes the frame against the reference words (for ``mixbf16`` the
    row-wise mix of two references with the candidate's coefficients, whose digest is
    checked), and the module receives a ``PredictiveContextTensor`` that resolves the
    references when it decodes.  A candidate stored transposed (``target transpose``: the real
    model's down projections, GCR/bitexact_predictive_serving.py:909-933) cannot be contracted by
    the tile walker as it lies; with ``reframe_transposed`` (the default) it is decoded once at load,
    turned and encoded row-major with the context codec, and that frame stays resident instead
    (``PredictiveContextTensor.reframe``; the receipt lists such tensors under
    ``reframed_tensors`` and counts them as transcoded), so its products are fused launches with
    no dense transient; off, it is decoded to a dense transient and multiplied by the library
    on every call, which is what the reference does with every frame.  ``share_launches`` names sibling linears that are applied to
    one tensor, e.g. ``[("q_proj", "k_proj", "v_proj"), ("gate_proj", "up_proj")]``: wherever a
    module has all the children of a tuple as coded linears of one input width (and the device
    tensors support it), they are indexed with one segment length and multiplied in one
    launch (``SharedProducts``); the receipt lists them under ``shared_launches``.
    ``batch_invariant=True`` is the M-invariant policy: every coded linear sends every row count
    through the matrix-core kernel, so a verify pass over k + 1 rows reproduces the one-row
    decode steps bit for bit (GS/miv_gemv.py:1-9); the default lets the row count pick the
    fastest kernel, and rows are then bit-equal only between calls of the same kernel family
    (``bitexact_context_gpu.route_rows``).  The receipt records the choice.  ``check_inventory``: check
    every file of the package against the manifest's ``files`` inventory (and the archive of the
    parent package's receipts) before anything is served; None does so when the manifest says
    ``verify_on_load``, as the reference's predictive packages do; ``optional_files`` names
    inventory paths that may be absent (the ``decoder/`` copies of the builder's sources, which
    this library does not use).  What this loader leaves to the caller is the model
    construction itself (the reference reads a Transformers config and generation config
    from the package's sidecars): ``model_factory`` returns the module to fill."""
    import hashlib
    from concurrent.futures import ThreadPoolExecutor, as_completed
    from pathlib import Path

    import numpy as np

    from . import bitexact_context_package as pkg
    if isinstance(loader_workers, bool) or not isinstance(loader_workers, int) or loader_workers < 1:
        raise ValueError("loader_workers must be a positive integer")
    if isinstance(dtype, str):
        dtype = getattr(torch, dtype)
    package = Path(package)
    try:
        manifest, entries = pkg.read_manifest(package)
        # the model's configuration sidecars are checked against their pins before any weight is read
        sidecars = pkg.read_metadata(package, manifest) if ("metadata_assets" in manifest or "files" in manifest) else {}
        # a package that asks for it is checked file by file before anything is served from it
        # (the reference's predictive loader runs its package verifier at load,
        # GCR/bitexact_predictive_serving.py:727-731)
        inventory_checked = manifest.get("verify_on_load") is True if check_inventory is None else bool(check_inventory)
        if inventory_checked:
            pkg.verify_inventory(package, manifest, optional=optional_files)
            pkg.verify_receipt_archive(package, manifest)
    except pkg.PackageError as exc:
        raise ContextServingError(str(exc)) from exc
    if tensor_factory is None:
        tensor_factory = hip_tensor_factory
    if predictive_factory is None:
        predictive_factory = hip_predictive_factory
    if mix_predictor is None:
        from .bitexact_predictive_mix import predict as mix_predictor
    if host_decoder is None:
        from .bitexact_context_codec import decode as host_decoder
    try:
        selected = pkg.read_candidates(package, manifest, entries)
    except pkg.PackageError as exc:
        raise ContextServingError(str(exc)) from exc

    previous = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device("meta"):
            model = model_factory()
    finally:
        torch.set_default_dtype(previous)

    try:
        params = dict(model.named_parameters(remove_duplicate=False))
    except TypeError:
        params = dict(model.named_parameters())
    if not params:
        raise ContextServingError("model has no named parameters")
    missing = sorted(set(params) - set(entries))
    if missing:
        raise ContextServingError(f"package missing required model parameters: {missing[:12]}")
    wrong = [(n, tuple(entries[n]["shape"]), tuple(p.shape)) for n, p in params.items()
             if tuple(entries[n]["shape"]) != tuple(p.shape)]
    if wrong:
        raise ContextServingError(f"manifest/model shape mismatch: {wrong[:8]}")

    def frame_of(name):
        try:
            return pkg.read_frame(package, entries[name])
        except pkg.PackageError as exc:
            raise ContextServingError(str(exc)) from exc

    def host_value(name, parameter):
        row = entries[name]
        decoded = host_decoder(frame_of(name))
        if isinstance(decoded, torch.Tensor):
            if decoded.dtype != torch.bfloat16:
                raise ContextServingError("host BCTX decoder did not return BF16")
            decoded = decoded.detach().cpu().contiguous().view(torch.uint16).numpy()
        if tuple(decoded.shape) != pkg.frame_shape(row["shape"]):
            raise ContextServingError(f"BCTX decoded frame geometry mismatch: {name}")
        if hashlib.sha256(decoded.astype("<u2", copy=False).tobytes()).hexdigest() != row["source_sha256"]:
            raise ContextServingError(f"BCTX decoded-source identity mismatch: {name}")
        runtime = _runtime_dtype(model, name, parameter, dtype)
        value = torch.from_numpy(decoded.copy()).view(torch.bfloat16).reshape(tuple(parameter.shape))
        return value.to(runtime).contiguous(), runtime

    def create_context(name):
        row = entries[name]
        extra = {"fused_segment": shared_segment[name]} if name in shared_segment and takes_segment else {}
        context = tensor_factory(frame_of(name), stride=stride, device=device, **extra)
        if tuple(context.shape) != pkg.frame_shape(row["shape"]):
            raise ContextServingError(f"indexed BCTX shape mismatch: {name}")
        if context.source_sha256 != row["source_sha256"]:
            raise ContextServingError(f"BCTX decoded-source identity mismatch: {name}")
        if getattr(context, "frame_sha256", None) != row["frame_sha256"]:
            raise ContextServingError(f"BCTX backend frame identity mismatch: {name}")
        resident = getattr(context, "resident_bytes", None)
        if type(resident) is not int or resident < 0:
            raise ContextServingError(f"BCTX backend lacks valid resident_bytes: {name}")
        return context, resident

    def record(name, kind, resident=0, **extra):
        row = selected.get(name) if kind.startswith("compressed") and name in selected else entries[name]
        return dict(kind=kind, shape=list(row["shape"]), source_sha256=row["source_sha256"],
                    frame_sha256=row["frame_sha256"], frame_bytes=row["frame_bytes"],
                    resident_context_bytes=resident, **extra)

    coded = [(module_name, module, f"{module_name}.weight" if module_name else "weight")
             for module_name, module in list(model.named_modules())
             if isinstance(module, (nn.Linear, nn.Embedding))]
    coded = [item for item in coded if item[2] in entries]

    # sibling linears that are to share a launch: found by attribute names under one parent
    import inspect
    try:
        takes_segment = "fused_segment" in inspect.signature(tensor_factory).parameters
    except (TypeError, ValueError):
        takes_segment = False
    try:
        predictive_takes_segment = "fused_segment" in inspect.signature(predictive_factory).parameters
    except (TypeError, ValueError):
        predictive_takes_segment = False
    # (predictive candidates too: siblings that are all coded against references, or all re-framed
    # at load, share launches like plain frames; mixed groups keep separate launches)
    coded_linears = {module_name: (module, weight_name) for module_name, module, weight_name in coded
                     if isinstance(module, nn.Linear)}
    sibling_groups, shared_segment = [], {}
    for names in share_launches or ():
        names = tuple(names)
        if not 2 <= len(names) <= 4:
            raise ValueError("share_launches: groups of 2..4 sibling names")
        for module_name in list(coded_linears):
            parent, _, attr = module_name.rpartition(".")
            if attr != names[0]:
                continue
            members = [f"{parent}.{n}" if parent else n for n in names]
            if all(m in coded_linears for m in members) and \
                    len({coded_linears[m][0].in_features for m in members}) == 1:
                sibling_groups.append(members)
                if takes_segment or predictive_takes_segment:
                    from . import _fused
                    cols = coded_linears[members[0]][0].in_features
                    try:
                        segment = _fused.choose_segment(cols, None, rows=max(coded_linears[m][0].out_features for m in members))
                    except _fused.FusedUnsupported:
                        continue
                    for m in members:
                        shared_segment[coded_linears[m][1]] = segment

    # tensors that need an object on the device: the coded weights and, transitively, the
    # references of predictive candidates; plain frames first (in parallel), then the
    # candidates in dependency order
    needed, order = set(), []

    def need(name):
        if name in needed:
            return
        needed.add(name)
        for ref in selected.get(name, {}).get("references", ()):
            need(ref["name"])
        order.append(name)

    for _, _, weight_name in coded:
        need(weight_name)
    plain = [name for name in order if name not in selected]
    contexts, done = {}, 0

    def accept(name, result):
        nonlocal done
        contexts[name] = result
        done += 1
        if done % 25 == 0 or done == len(order):
            log(f"[bctx] indexed {done}/{len(order)} compressed tensors")
            if progress_callback is not None:
                progress_callback(done, len(order), name)

    if loader_workers == 1:
        for name in plain:
            accept(name, create_context(name))
    elif plain:
        with ThreadPoolExecutor(max_workers=loader_workers, thread_name_prefix="bctx-index") as pool:
            futures = {pool.submit(create_context, name): name for name in plain}
            for future in as_completed(futures):
                accept(futures[future], future.result())

    host_words = {}  # frame-shaped uint16 words of references, dropped once the candidates are indexed

    def words_of(name):
        if name in host_words:
            return host_words[name]
        row = entries[name]
        if name in selected:
            from .bitexact_predictive_codec import decode as predictive_decode
            value = predictive_decode(candidate_frame(name), reference_words(name))
            if selected[name]["transform"] == "target transpose":
                value = value.T
        else:
            value = host_decoder(frame_of(name))
            if isinstance(value, torch.Tensor):
                value = value.detach().cpu().contiguous().view(torch.uint16).numpy()
        value = np.ascontiguousarray(value).reshape(pkg.frame_shape(row["shape"]))
        if hashlib.sha256(value.astype("<u2", copy=False).tobytes()).hexdigest() != row["source_sha256"]:
            raise ContextServingError(f"BCTX decoded-source identity mismatch: {name}")
        host_words[name] = value
        return value

    def candidate_frame(name):
        try:
            return pkg.read_candidate_frame(package, selected[name])
        except (pkg.PackageError, OSError) as exc:
            raise ContextServingError(str(exc)) from exc

    def reference_words(name):
        c = selected[name]
        refs = [words_of(ref["name"]) for ref in c["references"]]
        if c["mode"] == "single":
            return refs[0]
        derived = np.ascontiguousarray(mix_predictor(refs[0], refs[1], pkg.read_coefficients(package, c)), dtype="<u2")
        if hashlib.sha256(derived.tobytes()).hexdigest() != c["derived_reference_sha256"]:
            raise ContextServingError(f"derived reference checksum mismatch: {name}")
        return derived

    reframed = []
    for name in order:
        if name not in selected:
            continue
        c, row = selected[name], entries[name]
        extra = {"fused_segment": shared_segment[name]} if name in shared_segment and predictive_takes_segment else {}
        native = predictive_factory(candidate_frame(name), reference_words(name), stride=stride, device=device, **extra)
        geometry = pkg.frame_shape(row["shape"])
        if c["transform"] == "target transpose":
            geometry = geometry[::-1]
        if tuple(native.shape) != geometry:
            raise ContextServingError(f"PPCX frame geometry mismatch: {name}")
        if getattr(native, "frame_sha256", None) != c["frame_sha256"]:
            raise ContextServingError(f"PPCX frame identity mismatch: {name}")
        own = getattr(native, "resident_bytes", None)
        if type(own) is not int or own < 0:
            raise ContextServingError(f"PPCX resident byte accounting missing: {name}")
        coefficients = None
        if c["mode"] == "mixbf16":
            coefficients = torch.from_numpy(pkg.read_coefficients(package, c)).view(torch.bfloat16).to(device)
            own += coefficients.numel() * coefficients.element_size()
        wrapped = PredictiveContextTensor(
            native, [contexts[ref["name"]][0] for ref in c["references"]],
            predictor=mix_predictor if c["mode"] == "mixbf16" else None, coefficients=coefficients,
            transform=c["transform"], shape=pkg.frame_shape(row["shape"]), source_sha256=row["source_sha256"],
            frame_sha256=c["frame_sha256"], resident_bytes=own)
        if reframe_transposed and c["transform"] == "target transpose" and hasattr(native, "decode"):
            try:
                wrapped.reframe(tensor_factory, stride=stride, device=device)
                own = wrapped.resident_bytes
                reframed.append(name)
            except ContextServingError:
                raise
            except Exception as exc:  # the frame stays as it is: decode + dense product per call
                log(f"[bctx] {name}: not re-framed ({exc})")
        accept(name, (wrapped, own))
    host_words.clear()

    def residency(context):
        """What the device holds of a coded tensor, where the backend says so: the frame's mode,
        the mode of the resident form (a frame whose conditional residual stream was re-packed
        into 6-bit fields at load is resident in mode 0), and whether the fused kernels take it."""
        native = getattr(context, "row_major", None) or getattr(context, "native", context)
        if not hasattr(native, "resident_mode"):
            return {}
        fused = getattr(native, "fused", None) is not None
        reason = getattr(native, "fused_reason", "")
        return dict(frame_mode=native.mode, resident_mode=native.resident_mode,
                    residual_repacked=native.resident_mode != native.mode, fused=fused,
                    **({} if fused else {"fused_reason": reason}))

    consumed, replacements = {}, {}
    for module_name, module, weight_name in coded:
        context, resident = contexts[weight_name]
        extra = residency(context)
        if extra and not extra["fused"] and extra["frame_mode"] != 1:
            log(f"{weight_name}: decoded by the general kernel and multiplied densely ({extra['fused_reason']})")
        if isinstance(module, nn.Linear):
            bias = None
            if module.bias is not None:
                bias_name = f"{module_name}.bias" if module_name else "bias"
                if bias_name not in entries:
                    raise ContextServingError(f"package missing required linear bias: {bias_name}")
                value, runtime = host_value(bias_name, module.bias)
                bias = nn.Parameter(value, requires_grad=False)
                consumed[bias_name] = record(bias_name, "dense_bias", runtime_dtype=str(runtime))
            replacements[module_name] = BctxLinear(context, bias, batch_invariant=batch_invariant)
            consumed[weight_name] = record(weight_name, "compressed_linear", resident, **extra)
        else:
            replacements[module_name] = BctxEmbedding(context, padding_idx=module.padding_idx)
            consumed[weight_name] = record(weight_name, "compressed_embedding", resident, **extra)
    shared_launches = []
    for members in sibling_groups:
        modules = [replacements[m] for m in members]
        try:
            group = _launch_group([m.context_weight for m in modules])
            if group is None:
                continue
            products = SharedProducts(group, [m.bias for m in modules], batch_invariant=batch_invariant)
        except Exception as exc:  # the members stay separate launches
            log(f"[bctx] {members} keep separate launches: {exc}")
            continue
        for index, module in enumerate(modules):
            module.shared = (products, index)
        shared_launches.append([coded_linears[m][1] for m in members])
    # parents before children, so that a replaced parent is not looked up through a stale child
    for name, replacement in sorted(replacements.items(), key=lambda item: item[0].count(".")):
        parent, attr = _parent_and_attr(model, name)
        setattr(parent, attr, replacement)

    for name, parameter in params.items():
        if name in consumed:
            continue
        value, runtime = host_value(name, parameter)
        parent, attr = _parent_and_attr(model, name)
        parent._parameters[attr] = nn.Parameter(value, requires_grad=False)
        consumed[name] = record(name, "dense_parameter", runtime_dtype=str(runtime))

    left = [f"parameter:{n}" for n, p in model.named_parameters() if p.is_meta]
    left += [f"buffer:{n}" for n, b in model.named_buffers() if b.is_meta]
    if left:
        raise ContextServingError(f"model contains unfilled meta tensors: {left[:12]}")
    model.to(device)
    compressed = [n for n, r in consumed.items() if r["kind"].startswith("compressed")]
    receipt = {
        "schema": "georefine.bctx_serving_load.v1", "status": "ok", "format": "BCTX v1",
        "device": str(device), "dtype_default": str(dtype),
        "package_manifest": str(package / "manifest.json"), "verified_metadata_assets": sorted(sidecars),
        "tensor_count": len(entries), "consumed_count": len(consumed),
        "unused_package_tensors": sorted(set(entries) - set(consumed)),
        "compressed_tensor_count": len(compressed),
        "resident_context_bytes": sum(consumed[n]["resident_context_bytes"] for n in compressed),
        "dense_parameter_bytes": sum(p.numel() * p.element_size() for p in model.parameters()),
        "buffer_bytes": sum(b.numel() * b.element_size() for b in model.buffers()),
        "consumed_tensors": consumed, "restored_bf16_control": False,
        # true when a frame's residual stream is resident in another form than the frame's own
        # (re-packed 6-bit fields); the main stream and the decoded words are never altered
        "transcoded": any(r.get("residual_repacked") for r in consumed.values()) or bool(reframed),
        # predictive frames stored transposed that were decoded, turned and encoded row-major at load
        "reframed_tensors": sorted(reframed),
        "package_inventory_checked": inventory_checked,
        "residual_repacked_tensors": sorted(n for n, r in consumed.items() if r.get("residual_repacked")),
        "general_kernel_tensors": sorted(n for n, r in consumed.items()
                                         if r.get("fused") is False and r.get("frame_mode") != 1),
        "shared_launches": shared_launches,
        "batch_invariant": bool(batch_invariant),
    }
    return model, receipt


def load_predictive_model(package, *, model_factory, device="cuda:0", dtype=torch.bfloat16, stride=1024,
                          tensor_factory=None, context_factory=None, predictive_factory=None, mix_predictor=None,
                          host_decoder=None, loader_workers=1, batch_invariant=False, log=print,
                          progress_callback=None, share_launches=(), reframe_transposed=True, check_inventory=None,
                          optional_files=("decoder/",)):
    """The predictive-package loader under the reference's name and keywords
    (GCR/bitexact_predictive_serving.py:596-619): ``context_factory`` makes the BCTX tensors
    (``tensor_factory`` is accepted as its older spelling), ``predictive_factory`` the PPCX ones,
    ``mix_predictor`` the mixed references.  ``load_bctx_model`` already resolves the manifest's
    ``selected_candidates``, so both names load the same packages; this one insists that the
    package has candidates to resolve."""
    from . import bitexact_context_package as pkg
    if context_factory is not None and tensor_factory is not None and context_factory is not tensor_factory:
        raise ValueError("pass context_factory or tensor_factory, not two different ones")
    manifest, _ = pkg.read_manifest(package)
    if not manifest.get("selected_candidates"):
        raise ContextServingError("package has no predictive candidates; use load_bctx_model")
    return load_bctx_model(package, model_factory=model_factory, device=device, dtype=dtype, stride=stride,
                           tensor_factory=context_factory or tensor_factory, predictive_factory=predictive_factory,
                           mix_predictor=mix_predictor, host_decoder=host_decoder, loader_workers=loader_workers,
                           batch_invariant=batch_invariant, log=log, progress_callback=progress_callback,
                           share_launches=share_launches, reframe_transposed=reframe_transposed,
                           check_inventory=check_inventory, optional_files=optional_files)

