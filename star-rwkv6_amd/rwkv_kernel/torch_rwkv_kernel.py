"""torch flavour of the WKV6 operator: autograd.Function over libwkv6_gfx950.so.

Mirrors rwkv_kernel/torch_rwkv_kernel.py of the reference (constructor, call signature, argument
checks, 2-tuple return, dtype rules) but binds the library through its C ABI with ctypes instead
of JIT-building a torch C++ extension, and launches on torch's CURRENT stream.

Where the reference's torch flavour is broken as committed, the behaviour of its working
flavours is implemented: the default state_map for a single shared state has length batch
(ops_rwkv_kernal.py:54, against torch_rwkv_kernel.py:155), the stateful call actually runs
(torch_rwkv_kernel.py:93 names a binding that does not exist), and state_map is moved to the
device before the kernel reads it.
"""
import torch

from . import _native

_DTYPE_CODE = {torch.bfloat16: _native.BF16, torch.float16: _native.F16, torch.float32: _native.F32}


def _out_dtype(dt):
    # rwkv_kernel/torch_rwkv_kernel.py:35 -- float16 inputs produce float32 outputs
    return torch.float32 if dt == torch.float16 else dt


def _stream():
    return torch.cuda.current_stream().cuda_stream


_STAGGER = 256   # bytes


def _staggered(count, shape, dtype, device, first=1):
    """`count` tensors of one shape out of ONE allocation, the k-th starting (first + k) * 256 bytes
    past where a tensor of its own would start.  A workgroup of the kernels walks all (B,T,C) tensors
    of a call row by row in step; torch's allocator hands out large blocks on 2 MiB boundaries, and
    tensors whose bases agree modulo 4 KiB keep sending those streams to the same memory channel at
    the same moment (about 5 % of the training pair at B8 T1024 C2048).  The tensors are views of
    the common block, which lives as long as any of them."""
    n = 1
    for d in shape:
        n *= d
    es = torch.empty((), dtype=dtype).element_size()
    step = (n * es + _STAGGER - 1) // _STAGGER * _STAGGER + _STAGGER
    block = torch.empty(count * step + first * _STAGGER, dtype=torch.uint8, device=device)
    return [block[first * _STAGGER + i * step: first * _STAGGER + i * step + n * es].view(dtype).view(shape) for i in range(count)]


def _carve(device, specs):
    """Tensors of different shapes and dtypes out of ONE allocation: specs = [(shape, dtype, slot), ...]; each tensor
    starts `slot` * 256 bytes past a 4 KiB boundary of the block (see _staggered for why)."""
    offs, total = [], 0
    for shape, dtype, slot in specs:
        n = 1
        for d in shape:
            n *= d
        nb = n * _ELEMENT_SIZE[dtype]
        offs.append((total + slot * _STAGGER, nb))
        total += (slot * _STAGGER + nb + 4095) // 4096 * 4096
    block = torch.empty(total, dtype=torch.uint8, device=device)
    return [block[o:o + nb].view(dtype).view(shape) for (o, nb), (shape, dtype, _) in zip(offs, specs)]


_ELEMENT_SIZE = {torch.bfloat16: 2, torch.float16: 2, torch.float32: 4, torch.uint8: 1}
_saved_bytes_cache = {}


def _saved_bytes(lib, code, algo, B, T, C, H):
    key = (code, algo, B, T, C, H)
    n = _saved_bytes_cache.get(key)
    if n is None:
        n = _saved_bytes_cache[key] = int(lib.wkv6_saved_bytes(code, algo, B, T, C, H))
    return n


class _on_device:
    """torch.cuda.device(dev) only where dev is not already the current device (the context manager costs as much
    host time as a kernel launch)."""

    def __init__(self, dev):
        self.ctx = None if dev.index is None or dev.index == torch.cuda.current_device() else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


def _ptr(t):
    return None if t is None else t.data_ptr()


class _WKV6(torch.autograd.Function):
    """Stateless operator with gradients (rwkv_kernel/torch_rwkv_kernel.py:14-75).

    When a gradient will be needed and the library has something worth keeping for it (the chunked
    kernels' per-chunk states), the forward runs as wkv6_forward_save and the backward as
    wkv6_backward_saved; otherwise the plain pair the reference's binding corresponds to."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u, algo):
        lib = _native.load()
        with torch.no_grad():
            assert r.dtype == k.dtype == v.dtype == w.dtype == u.dtype
            assert r.dtype in _DTYPE_CODE
            for x in (r, k, v, w, u):
                assert x.is_contiguous()
            ctx.dims = (B, T, C, H)
            ctx.algo = algo
            code = _DTYPE_CODE[r.dtype]
            need_grad = any(ctx.needs_input_grad[4:9])
            nsave = _saved_bytes(lib, code, algo, B, T, C, H) if need_grad else 0
            saved = None
            if nsave:
                y, saved = _carve(r.device, [((B, T, C), _out_dtype(r.dtype), 5), ((nsave,), torch.uint8, 6)])
            else:
                (y,) = _staggered(1, (B, T, C), _out_dtype(r.dtype), r.device, first=5)
            with _on_device(r.device):
                if nsave:
                    _native.check(lib.wkv6_forward_save(_stream(), code, algo, B, T, C, H,
                                                        _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(y),
                                                        _ptr(saved), nsave))
                else:
                    # optional workspace: a long sequence of few (batch, head) pairs runs as time segments
                    n = lib.wkv6_forward_workspace_bytes(code, algo, B, T, C, H)
                    ws = torch.empty(int(n), device=r.device, dtype=torch.uint8) if n else None
                    _native.check(lib.wkv6_forward_ex(_stream(), code, algo, B, T, C, H,
                                                      _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(y), _ptr(ws), n))
            ctx.saved_states = saved
            ctx.save_for_backward(r, k, v, w, u)
            return y

    @staticmethod
    def backward(ctx, gy):
        lib = _native.load()
        assert gy.is_cuda
        with torch.no_grad():
            B, T, C, H = ctx.dims
            r, k, v, w, u = ctx.saved_tensors
            odt = _out_dtype(r.dtype)
            assert gy.dtype in (torch.bfloat16, torch.float32) and gy.dtype == odt
            gy = gy.contiguous()
            big = ((B, T, C), odt)
            gr, gk, gv, gw, gu, gu_sum = _carve(gy.device, [big + (7,), big + (8,), big + (9,), big + (10,),
                                                            ((B, C), odt, 0), ((C,), odt, 0)])
            code = _DTYPE_CODE[r.dtype]
            args = (_ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(gy), _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu))
            with _on_device(gy.device):
                saved = ctx.saved_states
                if saved is not None:
                    # the batch sum of gu (rwkv_kernel/torch_rwkv_kernel.py:73) comes out of the same launch
                    ctx.saved_states = None
                    _native.check(lib.wkv6_backward_saved_sum(_stream(), code, ctx.algo, B, T, C, H, *args, _ptr(gu_sum),
                                                              _ptr(saved), saved.numel()))
                    return (None, None, None, None, gr, gk, gv, gw, gu_sum.reshape(u.shape), None)
                else:
                    ws_bytes = lib.wkv6_backward_workspace_bytes_ex(code, ctx.algo, B, T, C, H)
                    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=gy.device) if ws_bytes else None
                    _native.check(lib.wkv6_backward_ex(_stream(), code, ctx.algo, B, T, C, H, *args, _ptr(ws), ws_bytes))
            # per-batch partials -> shape of u, rwkv_kernel/torch_rwkv_kernel.py:73
            gu = torch.sum(gu, 0).reshape(u.shape)
            return (None, None, None, None, gr, gk, gv, gw, gu, None)


class _WKV6GnGate(torch.autograd.Function):
    """out = (group_norm_head(wkv6(r, k, v, w, u)) * gn_scale + gn_offset) * gate with gradients, bf16,
    zero initial state: the operator and what the layer does with its output next
    (rwkv6_model.py:94-99,158-160) in one forward kernel (wkv6_forward_gn_gate_save: y never makes the
    trip to the norm's own kernels and back), the norm's and the gate's backward in one elementwise
    kernel (wkv6_gn_gate_backward), then the operator's backward from the saved chunk states."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u, gate, gn_scale, gn_offset, eps):
        lib = _native.load()
        with torch.no_grad():
            code = _DTYPE_CODE[r.dtype]
            sc = gn_scale.detach().to(dtype=torch.float32).contiguous()
            of = gn_offset.detach().to(dtype=torch.float32).contiguous()
            out, y = _staggered(2, (B, T, C), r.dtype, r.device, first=5)
            stats = torch.empty((B, T, H, 2), device=r.device, dtype=torch.float32)
            with torch.cuda.device(r.device):
                nsave = lib.wkv6_saved_bytes(code, _native.ALGO_CHUNK, B, T, C, H)
                (saved,) = _staggered(1, (nsave,), torch.uint8, r.device, first=7)
                _native.check(lib.wkv6_forward_gn_gate_save(
                    _stream(), code, B, T, C, H, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(gate), _ptr(sc), _ptr(of),
                    float(eps), _ptr(out), _ptr(y), _ptr(stats), _ptr(saved), nsave))
            ctx.dims = (B, T, C, H)
            ctx.saved_states = saved
            ctx.save_for_backward(r, k, v, w, u, gate, sc, of, y, stats)
            ctx.param_shapes = (gn_scale.shape, gn_offset.shape, gn_scale.dtype, gn_offset.dtype)
            return out

    @staticmethod
    def backward(ctx, gout):
        lib = _native.load()
        with torch.no_grad():
            B, T, C, H = ctx.dims
            r, k, v, w, u, gate, sc, of, y, stats = ctx.saved_tensors
            saved, ctx.saved_states = ctx.saved_states, None
            assert gout.dtype == r.dtype
            gout = gout.contiguous()
            code = _DTYPE_CODE[r.dtype]
            gy, ggate = _staggered(2, (B, T, C), r.dtype, r.device, first=5)
            gr, gk, gv, gw = _staggered(4, (B, T, C), r.dtype, r.device, first=7)
            gsc = torch.empty(C, device=r.device, dtype=torch.float32)
            gof = torch.empty(C, device=r.device, dtype=torch.float32)
            gu = torch.empty((B, C), device=r.device, dtype=r.dtype)
            gu_sum = torch.empty(C, device=r.device, dtype=r.dtype)
            with torch.cuda.device(r.device):
                _native.check(lib.wkv6_gn_gate_backward(_stream(), code, B, T, C, H, _ptr(gout), _ptr(y), _ptr(stats), _ptr(gate),
                                                        _ptr(sc), _ptr(of), _ptr(gy), _ptr(ggate), _ptr(gsc), _ptr(gof)))
                if saved is not None:
                    _native.check(lib.wkv6_backward_saved_sum(_stream(), code, _native.ALGO_CHUNK, B, T, C, H,
                                                              _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(gy),
                                                              _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu), _ptr(gu_sum),
                                                              _ptr(saved), saved.numel()))
                else:
                    # a second backward over the same graph (retain_graph): the saved block went with the
                    # first one (its counters are used up); the plain backward rebuilds the states itself
                    ws_bytes = lib.wkv6_backward_workspace_bytes_ex(code, _native.ALGO_CHUNK, B, T, C, H)
                    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device) if ws_bytes else None
                    _native.check(lib.wkv6_backward_ex(_stream(), code, _native.ALGO_CHUNK, B, T, C, H,
                                                       _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(gy),
                                                       _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu), _ptr(ws), ws_bytes))
                    gu_sum = torch.sum(gu, 0)
            s_shape, o_shape, s_dt, o_dt = ctx.param_shapes
            return (None, None, None, None, gr, gk, gv, gw, gu_sum.reshape(u.shape), ggate,
                    gsc.reshape(s_shape).to(s_dt), gof.reshape(o_shape).to(o_dt), None)


class _ShiftMix(torch.autograd.Function):
    """The layer's input side (rwkv6_model.py:134-146) with gradients, bf16: x -> (xr, xk, xv, xw, xg).
    Token shift and x_mix in one kernel (wkv6_shift_mix_x), the GEMM against the stacked first mixer
    weights and its tanh in torch, then one kernel that expands the rank-R coefficients on the matrix
    cores and writes the five outputs (wkv6_shift_mix_five).  Backward: wkv6_shift_mix_five_backward,
    the reductions over channels and over tokens as batched GEMMs, wkv6_shift_mix_x_backward."""

    @staticmethod
    def forward(ctx, x, mix_x, a, w2t, bias):
        lib = _native.load()
        with torch.no_grad():
            B, T, C = x.shape
            R = w2t.shape[2]
            code = _DTYPE_CODE[x.dtype]
            mx = mix_x.detach().to(torch.float32).contiguous()
            a16 = a.detach().to(x.dtype).contiguous()
            w16 = w2t.detach().to(x.dtype).contiguous()
            b32 = bias.detach().to(torch.float32).contiguous()
            x_mix = torch.empty_like(x)
            outs = _staggered(5, (B, T, C), x.dtype, x.device, first=1)
            with torch.cuda.device(x.device):
                _native.check(lib.wkv6_shift_mix_x(_stream(), code, B, T, C, _ptr(x), _ptr(mx), _ptr(x_mix)))
                h = torch.tanh(x_mix.view(B * T, C) @ a16.t())            # (B*T, 5R)
                _native.check(lib.wkv6_shift_mix_five(_stream(), code, B, T, C, R, _ptr(x), _ptr(h), _ptr(w16), _ptr(b32),
                                                      *[_ptr(o) for o in outs]))
            ctx.save_for_backward(x, x_mix, h, mx, a16, w16, b32)
            ctx.param_dtypes = (mix_x.dtype, a.dtype, w2t.dtype, bias.dtype)
            return tuple(outs)

    @staticmethod
    def backward(ctx, *gouts):
        lib = _native.load()
        with torch.no_grad():
            x, x_mix, h, mx, a16, w16, b32 = ctx.saved_tensors
            B, T, C = x.shape
            n, R = B * T, w16.shape[2]
            code = _DTYPE_CODE[x.dtype]
            gouts = [torch.zeros_like(x) if g is None else g.to(x.dtype).contiguous() for g in gouts]
            # the five planes of gcoef 256 bytes further apart than they are long (see _staggered)
            plane = n * C + _STAGGER // 2
            gcoef = torch.empty(5 * plane, device=x.device, dtype=x.dtype).as_strided((5, n, C), (plane, C, 1))
            gp, gxx, gx = _staggered(3, (B, T, C), x.dtype, x.device, first=1)
            gmx = torch.empty(C, device=x.device, dtype=torch.float32)
            with torch.cuda.device(x.device):
                _native.check(lib.wkv6_shift_mix_five_backward(
                    _stream(), code, B, T, C, R, _ptr(x), _ptr(h), _ptr(w16), _ptr(b32), *[_ptr(g) for g in gouts],
                    _ptr(gcoef), plane, _ptr(gp), _ptr(gxx)))
                gh = torch.bmm(gcoef, w16)                                   # (5, n, R): summed over channels
                # sums over tokens: gcoef^T h for the weights and, through eight more columns of which
                # the first holds ones, gcoef^T 1 for the biases -- one pass over gcoef for both
                h3 = torch.zeros((5, n, R + 8), device=x.device, dtype=x.dtype)
                h3[:, :, :R] = h.view(n, 5, R).permute(1, 0, 2)
                h3[:, :, R] = 1
                gwb = torch.bmm(gcoef.transpose(1, 2), h3)                   # (5, C, R + 8)
                gw2t, gbias = gwb[:, :, :R], gwb[:, :, R]
                gpre = (gh.permute(1, 0, 2).reshape(n, 5 * R).float() * (1.0 - h.float() ** 2)).to(x.dtype)
                ga = gpre.t() @ x_mix.view(n, C)                             # (5R, C)
                gxm = (gpre @ a16).view(B, T, C)
                _native.check(lib.wkv6_shift_mix_x_backward(_stream(), code, B, T, C, _ptr(x), _ptr(mx), _ptr(gp), _ptr(gxx),
                                                            _ptr(gxm), _ptr(gx), _ptr(gmx)))
            dm, da, dw, db = ctx.param_dtypes
            return gx, gmx.to(dm), ga.to(da), gw2t.to(dw), gbias.to(db)


class _ShiftMixX(torch.autograd.Function):
    """x + (previous token - x) * mix with gradients, bf16 (wkv6_shift_mix_x and its backward): the fixed
    token-shift mix of rwkv6_model.py:136 (time mix) and :57-60 (channel mix)."""

    @staticmethod
    def forward(ctx, x, mix):
        lib = _native.load()
        with torch.no_grad():
            B, T, C = x.shape
            mx = mix.detach().to(torch.float32).contiguous()
            out = torch.empty_like(x)
            with torch.cuda.device(x.device):
                _native.check(lib.wkv6_shift_mix_x(_stream(), _DTYPE_CODE[x.dtype], B, T, C, _ptr(x), _ptr(mx), _ptr(out)))
            ctx.save_for_backward(x, mx)
            ctx.mix_dtype = mix.dtype
            return out

    @staticmethod
    def backward(ctx, gout):
        lib = _native.load()
        with torch.no_grad():
            x, mx = ctx.saved_tensors
            B, T, C = x.shape
            gout = gout.to(x.dtype).contiguous()
            gx = torch.empty_like(x)
            gmx = torch.empty(C, device=x.device, dtype=torch.float32)
            with torch.cuda.device(x.device):
                _native.check(lib.wkv6_shift_mix_x_backward(_stream(), _DTYPE_CODE[x.dtype], B, T, C, _ptr(x), _ptr(mx), None, None,
                                                            _ptr(gout), _ptr(gx), _ptr(gmx)))
            return gx, gmx.to(ctx.mix_dtype)


def _forward_with_state(B, T, C, H, state_map, r, k, v, w, u, init_state, algo=_native.ALGO_AUTO, state_dtype=None):
    """Stateful forward, no gradient (rwkv_kernel/torch_rwkv_kernel.py:76-95)."""
    lib = _native.load()
    with torch.no_grad():
        # state_map None with an init_state means the identity map (row b starts from init_state[b])
        assert init_state is not None or state_map is None, "state_map needs init_state"
        assert state_map is None or state_map.dtype == torch.int64
        odt = _out_dtype(r.dtype)
        sdt = init_state.dtype if init_state is not None else (state_dtype or odt)
        N = C // H
        (y,) = _staggered(1, (B, T, C), odt, r.device, first=5)
        ys = torch.empty((B, H, N, N), device=r.device, dtype=sdt)
        with torch.cuda.device(r.device):
            # optional workspace: lets a long sequence of few (batch, head) pairs run as time segments
            n = lib.wkv6_forward_workspace_bytes(_DTYPE_CODE[r.dtype], algo, B, T, C, H)
            ws = torch.empty(int(n), device=r.device, dtype=torch.uint8) if n else None
            _native.check(lib.wkv6_forward_with_state_ex(
                _stream(), _DTYPE_CODE[r.dtype], _DTYPE_CODE[sdt], algo, B, T, C, H,
                int(init_state is not None), _ptr(state_map),
                _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(init_state), _ptr(y), _ptr(ys), _ptr(ws), n))
    return y, ys


class _WKV6State(torch.autograd.Function):
    """Stateful operator WITH gradients through the state: y, S_T = f(r, k, v, w, u, S_0), states fp32
    (B,H,N,N), one per batch row.  Not part of the reference, whose stateful call carries no gradient
    (rwkv_kernel/torch_rwkv_kernel.py:145-168); it makes back-propagation over a sequence cut into
    pieces possible (the state's gradient is handed from one piece to the one before)."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u, s0, algo):
        ctx.dims = (B, T, C, H)
        ctx.algo = algo
        ctx.has_s0 = s0 is not None
        ctx.set_materialize_grads(False)   # an unused output arrives as None, not as a tensor of zeros
        y, sT = _forward_with_state(B, T, C, H, None, r, k, v, w, u, s0, algo, state_dtype=torch.float32)
        ctx.save_for_backward(r, k, v, w, u, *((s0,) if s0 is not None else ()))
        return y, sT

    @staticmethod
    def backward(ctx, gy, gsT):
        B, T, C, H = ctx.dims
        r, k, v, w, u = ctx.saved_tensors[:5]
        s0 = ctx.saved_tensors[5] if ctx.has_s0 else None
        with torch.no_grad():
            odt = _out_dtype(r.dtype)
            gy = torch.zeros((B, T, C), device=r.device, dtype=odt) if gy is None else gy.to(odt).contiguous()
            gsT = None if gsT is None else gsT.float().contiguous()
            gr, gk, gv, gw, gu, gs0 = _backward_with_state(B, T, C, H, r, k, v, w, u, s0, gy, gsT, ctx.algo, ctx.has_s0)
            gu = torch.sum(gu, 0).reshape(u.shape)
        return (None, None, None, None, gr.to(r.dtype), gk.to(r.dtype), gv.to(r.dtype), gw.to(r.dtype), gu.to(u.dtype), gs0, None)


def _backward_with_state(B, T, C, H, r, k, v, w, u, s0, gy, gsT, algo, want_gs0):
    """gr, gk, gv, gw, per-row gu (B, C), dL/dS_0 or None, through wkv6_backward_with_state."""
    lib = _native.load()
    odt = _out_dtype(r.dtype)
    gr, gk, gv, gw = _staggered(4, (B, T, C), odt, r.device, first=7)
    gu = torch.empty((B, C), device=r.device, dtype=odt)
    gs0 = torch.empty((B, H, C // H, C // H), device=r.device, dtype=torch.float32) if want_gs0 else None
    code = _DTYPE_CODE[r.dtype]
    with torch.cuda.device(r.device):
        n = lib.wkv6_backward_with_state_workspace_bytes(code, algo, B, T, C, H)
        ws = torch.empty(max(int(n), 16), device=r.device, dtype=torch.uint8)
        _native.check(lib.wkv6_backward_with_state(
            _stream(), code, algo, B, T, C, H, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(s0),
            _ptr(gy), _ptr(gsT), _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu), _ptr(gs0), _ptr(ws), n))
    return gr, gk, gv, gw, gu, gs0


class RWKVKernelOperator:
    def __init__(self, head_size, max_sequence_length):
        lib = _native.load()
        assert isinstance(head_size, int) and isinstance(max_sequence_length, int)
        assert head_size > 0 and max_sequence_length > 0
        assert head_size % 4 == 0, "head_size must be a multiple of 4"
        if not lib.wkv6_supports_head_size(head_size):
            raise _native.WKV6Error("libwkv6_gfx950 is built for head sizes 64 (all paths) and the other multiples of 4 up to 128 (plain calls), got %d" % head_size)
        self.head_size = head_size
        # the reference bakes this into a per-thread array bound (-D_T_); nothing here is sized by
        # it, so longer sequences simply work
        self.max_sequence_length = max_sequence_length
        self.algo = _native.ALGO_AUTO
        self._zero_maps = {}
        self.normal_kernenl = _WKV6
        self.kernel_with_state = _forward_with_state

    def _check(self, r, k, v, w, u, init_state, state_map):
        """Argument checks shared by every entry; returns (B, T, C, H, N, u, init_state, state_map)."""
        B, T, C = r.shape
        N = self.head_size
        assert C % N == 0
        H = C // N
        if not isinstance(u, torch.Tensor):
            u = u.value

        for x in (r, k, v, w, u):
            assert x.is_cuda
        assert r.device == k.device == v.device == w.device == u.device
        assert r.dtype == k.dtype == v.dtype == w.dtype == u.dtype
        assert r.shape == k.shape == v.shape == w.shape
        assert u.numel() == C, "u must hold one value per channel"

        if init_state is not None:
            assert init_state.dim() in (3, 4), \
                "init_state must be (state_kinds <= batch, H, N, N) or (H, N, N)"
            if init_state.dim() == 3:
                init_state = init_state[None, :]
            assert tuple(init_state.shape[1:]) == (H, N, N) and init_state.shape[0] <= B, \
                "init_state must be (state_kinds <= batch, H, N, N) or (H, N, N)"
            s_dtype = _out_dtype(r.dtype)
            assert init_state.dtype in (s_dtype, torch.float32), "init_state dtype must be %s" % s_dtype
            assert init_state.device == r.device

        if state_map is not None:
            if isinstance(state_map, (list, tuple)):
                state_map = torch.tensor(state_map, dtype=torch.int64)
            elif isinstance(state_map, torch.Tensor):
                assert state_map.dtype in (torch.int32, torch.int64), "state_map must be int32/int64 of shape (batch,)"
                state_map = state_map.to(torch.int64)
            assert tuple(state_map.shape) == (B,), "state_map must have shape (batch,)"
        return B, T, C, H, N, u, init_state, state_map

    def _resolve_state(self, B, r, init_state, state_map):
        """Default / validated state_map on the device (None = identity), contiguous init_state."""
        if init_state is None:
            assert state_map is None, "state_map needs init_state"
            return None, None
        n_state = init_state.shape[0]
        if state_map is None:
            assert n_state == 1 or n_state == B, "cannot infer state_map; pass it explicitly"
            if n_state == 1 and B > 1:
                key = (B, r.device)
                if key not in self._zero_maps:
                    self._zero_maps[key] = torch.zeros(B, dtype=torch.int64, device=r.device)
                state_map = self._zero_maps[key]
            # n_state == B: identity, expressed as "no map" so that a decode loop pays
            # neither a host-to-device copy nor a range check per step
        else:
            assert bool((state_map >= 0).all()) and bool((state_map < n_state).all()), \
                "state_map values must lie in [0, %d)" % n_state
            state_map = state_map.to(r.device).contiguous()
        return init_state.contiguous(), state_map

    def __call__(self, r, k, v, w, u, return_state=False, init_state=None, state_map=None):
        B, T, C, H, N, u, init_state, state_map = self._check(r, k, v, w, u, init_state, state_map)
        if return_state:
            init_state, state_map = self._resolve_state(B, r, init_state, state_map)
            for x in (r, k, v, w, u):
                assert x.is_contiguous()
            leaves = (r, k, v, w, u) + ((init_state,) if init_state is not None else ())
            if torch.is_grad_enabled() and any(x.requires_grad for x in leaves):
                # gradients through the state (not in the reference): one fp32 state per batch row
                assert state_map is None and (init_state is None or init_state.shape[0] == B), \
                    "gradients through the state need one init_state row per batch row and no state_map"
                assert init_state is None or init_state.dtype == torch.float32, \
                    "gradients through the state need an fp32 init_state"
                return _WKV6State.apply(B, T, C, H, r, k, v, w, u, init_state, self.algo)
            return _forward_with_state(B, T, C, H, state_map, r, k, v, w, u, init_state, self.algo)
        o = _WKV6.apply(B, T, C, H, r, k, v, w, u, self.algo)
        return o, None

    def shift_mix_supported(self, x, decomposer_size):
        """Whether ``shift_mix`` takes this tensor (bf16 on the GPU, rank 32 or 64)."""
        if not (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 3):
            return False
        return bool(_native.load().wkv6_shift_mix_supported(_DTYPE_CODE[x.dtype], x.shape[2], decomposer_size))

    def shift_mix_x(self, x, mix):
        """``x + (previous token - x) * mix`` (zero before a sequence's first token), differentiable in both
        arguments: the fixed token-shift mix of rwkv6_model.py:136 and of the channel-mix layer
        (:57-60).  bf16 tensors on the GPU, ``mix`` one value per channel.  Not part of the reference's operator."""
        assert x.is_contiguous() and x.dim() == 3 and mix.numel() == x.shape[2]
        assert self.shift_mix_supported(x, 32), "shift_mix_x takes bf16 tensors on the GPU, channels a multiple of 64"
        return _ShiftMixX.apply(x, mix.reshape(x.shape[2]))

    def shift_mix(self, x, mix_x, a, w2t, bias):
        """The layer's input side, rwkv6_model.py:134-146: from the layer input ``x`` (B,T,C) to the
        inputs ``(xr, xk, xv, xw, xg)`` of the projections that produce r, k, v, w and the gate:
        ``x_s = x + xx * (tanh((x + xx * mix_x) a_s^T) w2t_s^T + bias_s)`` with ``xx`` the previous token
        minus the token.  ``a`` (5R, C): the five mixers' first weights stacked in the order r, k, v, w, g;
        ``w2t`` (5, C, R) and ``bias`` (5, C): their second weights and biases.  Differentiable in all
        five arguments.  Not part of the reference's operator."""
        B, T, C = x.shape
        assert x.is_contiguous() and mix_x.numel() == C
        R = w2t.shape[2]
        assert a.shape == (5 * R, C) and w2t.shape == (5, C, R) and bias.shape == (5, C)
        assert self.shift_mix_supported(x, R), "shift_mix takes bf16 tensors on the GPU with rank 32 or 64"
        return _ShiftMix.apply(x, mix_x.reshape(C), a, w2t, bias)

    def forward_gn_gate(self, r, k, v, w, u, gate, gn_scale, gn_offset, epsilon=64e-5,
                        return_state=False, init_state=None, state_map=None):
        """Forward with the layer's next two steps fused into the kernel's output stage: returns
        ``(group_norm(y) * gate, state)`` where group_norm is the per-head layer norm with scale and
        offset of rwkv6_model.py:94-99 and ``* gate`` is rwkv6_model.py:158-160.  bf16 tensors;
        gn_scale / gn_offset hold one value per channel.  Without gradients (inference) y itself is
        never written and the stateful arguments work as in ``__call__``.  With gradients enabled and
        required (training; no state arguments) the call is differentiable in r, k, v, w, u, gate,
        gn_scale and gn_offset.  Not part of the reference's operator."""
        B, T, C, H, N, u, init_state, state_map = self._check(r, k, v, w, u, init_state, state_map)
        assert r.dtype == torch.bfloat16, "the fused output stage takes bf16 tensors"
        assert gate.shape == r.shape and gate.dtype == r.dtype and gate.device == r.device
        assert gn_scale.numel() == C and gn_offset.numel() == C
        if torch.is_grad_enabled() and any(x.requires_grad for x in (r, k, v, w, u, gate, gn_scale, gn_offset)):
            assert not return_state and init_state is None and state_map is None, \
                "the differentiable fused call takes no state arguments"
            for x in (r, k, v, w, u, gate):
                assert x.is_contiguous()
            lib = _native.load()
            if lib.wkv6_forward_gn_gate_save_supported(_DTYPE_CODE[r.dtype], B, T, C, H):
                return _WKV6GnGate.apply(B, T, C, H, r, k, v, w, u, gate, gn_scale.to(r.device), gn_offset.to(r.device), epsilon), None
            # (a shape the fused training kernels do not take, e.g. a sequence too long for the chunk form: unfused calls)
            y, _ = self(r, k, v, w, u)
            z = torch.nn.functional.layer_norm(y.float().view(B, T, H, N), (N,), eps=epsilon).view(B, T, C)
            out = (z * gn_scale.reshape(1, 1, C).float() + gn_offset.reshape(1, 1, C).float()) * gate.float()
            return out.to(r.dtype), None
        init_state, state_map = self._resolve_state(B, r, init_state, state_map)
        for x in (r, k, v, w, u, gate):
            assert x.is_contiguous()
        lib = _native.load()
        with torch.no_grad():
            sc = gn_scale.detach().to(device=r.device, dtype=torch.float32).contiguous()
            of = gn_offset.detach().to(device=r.device, dtype=torch.float32).contiguous()
            sdt = init_state.dtype if init_state is not None else torch.float32
            out = torch.empty_like(r)
            ys = torch.empty((B, H, N, N), device=r.device, dtype=sdt) if return_state else None
            with torch.cuda.device(r.device):
                # optional workspace: a long sequence of few (batch, head) pairs runs as time segments
                n = lib.wkv6_forward_workspace_bytes(_DTYPE_CODE[r.dtype], _native.ALGO_CHUNK, B, T, C, H)
                ws = torch.empty(int(n), device=r.device, dtype=torch.uint8) if n else None
                _native.check(lib.wkv6_forward_gn_gate_ex(
                    _stream(), _DTYPE_CODE[r.dtype], _DTYPE_CODE[sdt], B, T, C, H,
                    int(init_state is not None), _ptr(state_map),
                    _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(init_state), _ptr(gate), _ptr(sc), _ptr(of),
                    float(epsilon), _ptr(out), _ptr(ys), _ptr(ws), n))
        return out, ys
