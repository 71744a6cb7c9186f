"""A small layer-table format for chained int8 networks and a runner that executes it on the
GPU through the C API (what generated deployment code does by hand with the reference:
one pulp_nn_* call per layer on caller-owned buffers).

A network is a list of layer dicts.  Every layer has "op", "name" and "in" (the name of the
tensor it reads; the network input is called "input"; "add" takes a pair of names) and
produces the tensor called like the layer.  Activations are HWC uint8, batch outermost.

  op            parameters
  conv          w [Co,ky,kx,Ci] int8, bias [Co] int8 or None, pads (t,b,l,r), strides (sx,sy),
                requantisation (below)                      -> pulp_nn_conv_Ho_parallel
  pointwise     w [Co,1,1,Ci], bias, requantisation        -> pulp_nn_pointwise_HoWo_parallel
  depthwise     w [C,ky,kx], bias, pads, strides, requantisation.  The tensor it reads is HWC
                like all others; the runner changes the layout (pulp_nn_hip_hwc_to_chw +
                pulp_nn_depthwise_generic) or, for 3x3 / padding 1 layers the library has a
                fused kernel for, calls pulp_nn_hip_depthwise_hwc; if the next layer is a
                pointwise layer that is the only reader of the depthwise result, the two run
                as one launch (pulp_nn_hip_dw_pw_hwc) and the depthwise result is not
                materialised: Runner(..., fuse_blocks=True) for every such pair, False for none,
                "auto" (the default) where it is not slower: as Runner.tune() measured it on the
                batch at hand, else for blocks whose output plane is 8 x 8 pixels
  maxpool       kernel (kx,ky), strides, pads, out_hw      -> pulp_nn_maxpool
  avgpool       kernel, strides, pads, out_hw, lam, shift, add, requant -> pulp_nn_avgpool
  add           in = (a, b), m1, m2, shift                 -> pulp_nn_add
  linear        w [N,K] int8, bias, requantisation; reads its input flattened per image
                                                           -> pulp_nn_linear
  linear_out_32 w [N,K], bias32 [N] int32 or None; int32 output -> pulp_nn_linear_out_32

Requantisation keys: relu, bn (the two flags), k, lam ([Co] arrays for bn), mult (out_mult),
shift (out_shift).  shift = None on a bn layer means "to be calibrated": Runner.calibrate()
sets it to floor(log2(max |acc * k|)) - 7 over the batch it is given, computed on the GPU
(pulp_nn_hip_calib_conv / pulp_nn_hip_calib_depthwise), layer by layer along the chain.
"""
import numpy as np

from .api import PulpNNError

CONV_LIKE = ("conv", "pointwise", "depthwise", "linear")


def out_size(n, k, s, p0, p1):
    return (n + p0 + p1 - k) // s + 1


def infer_shapes(layers, input_shape):
    """{tensor name: (H, W, C)} for the input and every layer output (linear outputs are (1, 1, N))."""
    shapes = {"input": tuple(input_shape)}
    for L in layers:
        op = L["op"]
        src = L["in"][0] if op == "add" else L["in"]
        H, W, Cc = shapes[src]
        if op in ("conv", "pointwise"):
            Co, ky, kx, Ci = L["w"].shape
            assert Ci == Cc, (L["name"], Ci, Cc)
            if op == "pointwise":
                shapes[L["name"]] = (H, W, Co)
            else:
                pt, pb, pl, pr = L["pads"]
                sx, sy = L["strides"]
                shapes[L["name"]] = L.get("out_hw", (out_size(H, ky, sy, pt, pb), out_size(W, kx, sx, pl, pr))) + (Co,)
        elif op == "depthwise":
            Cw, ky, kx = L["w"].shape
            assert Cw == Cc, (L["name"], Cw, Cc)
            pt, pb, pl, pr = L["pads"]
            sx, sy = L["strides"]
            shapes[L["name"]] = L.get("out_hw", (out_size(H, ky, sy, pt, pb), out_size(W, kx, sx, pl, pr))) + (Cc,)
        elif op in ("maxpool", "avgpool"):
            shapes[L["name"]] = tuple(L["out_hw"]) + (Cc,)
        elif op == "add":
            assert shapes[L["in"][1]] == (H, W, Cc), L["name"]
            shapes[L["name"]] = (H, W, Cc)
        elif op in ("linear", "linear_out_32"):
            N, K = L["w"].shape
            assert K == H * W * Cc, (L["name"], K, H * W * Cc)
            shapes[L["name"]] = (1, 1, N)
        else:
            raise ValueError("unknown op %r" % op)
    return shapes


class Runner:
    """Uploads the parameters once, owns the activation buffers and queues the chain."""

    def __init__(self, nn, layers, input_shape, batch, fused=True, fuse_blocks="auto", chain_blocks=True):
        import torch
        self.nn, self.layers, self.batch, self.torch = nn, layers, batch, torch
        self.fused, self.unfused = fused, set()
        self.fuse_blocks, self.unfused_blocks, self.launches = fuse_blocks, set(), 0
        self.block_choice = {}   # layer index of a depthwise layer -> run it and its pointwise layer as one launch (tune())
        # runs of depthwise + pointwise blocks of one shape as one launch each (pulp_nn_hip_dw_pw_chain_hwc)
        self.chain_blocks, self.unchained = bool(chain_blocks and fused and fuse_blocks), set()
        self.shapes = infer_shapes(layers, input_shape)
        bn_np = np.int64 if nn.bn_bits == 64 else np.int32

        def dev(a, dtype=None):
            return None if a is None else torch.from_numpy(np.ascontiguousarray(a, dtype=dtype)).cuda()

        self.params = []
        for L in layers:
            P = {}
            if "w" in L:
                P["w"] = dev(L["w"], np.int8)
            if L["op"] == "linear_out_32":
                P["bias"] = dev(L.get("bias32"), np.int32)
            elif "bias" in L:
                P["bias"] = dev(L["bias"], np.int8)
            if L.get("k") is not None:
                P["k"], P["lam"] = dev(L["k"], bn_np), dev(L["lam"], bn_np)
            self.params.append(P)
        self.act = {}
        for L in layers:
            H, W, Cc = self.shapes[L["name"]]
            dt = torch.int32 if L["op"] == "linear_out_32" else torch.uint8
            self.act[L["name"]] = torch.empty((batch, H, W, Cc), dtype=dt, device="cuda")
        self.chw = {}
        for L in layers:
            if L["op"] == "depthwise":
                H, W, Cc = self.shapes[L["in"]]
                self.chw[L["name"]] = torch.empty((batch, Cc, H, W), dtype=torch.uint8, device="cuda")
        self._calib = None

    # -- one layer ------------------------------------------------------------------------
    def _requant_args(self, L, P):
        relu, bn = L.get("relu", 0), L.get("bn", 0)
        if relu and bn and L.get("shift") is None:
            raise ValueError("layer %s has no out_shift: run calibrate() first" % L["name"])
        return P.get("k"), P.get("lam"), L.get("mult", 0), L.get("shift", 0) or 0, relu, bn

    def _queue(self, i, tensors):
        L, P, nn = self.layers[i], self.params[i], self.nn
        op, out = L["op"], self.act[L["name"]]
        if op == "add":
            a, b = tensors[L["in"][0]], tensors[L["in"][1]]
            H, W, Cc = self.shapes[L["name"]]
            nn.pulp_nn_add(a, b, out, L["m1"], L["m2"], L["shift"], H, W, Cc)
            return out
        cur = tensors[L["in"]]
        H, W, Cc = self.shapes[L["in"]]
        Ho, Wo, Co = self.shapes[L["name"]]
        if op in ("conv", "pointwise"):
            k, lam, mult, shift, relu, bn = self._requant_args(L, P)
            if op == "conv":
                ky, kx = L["w"].shape[1:3]
                pt, pb, pl, pr = L["pads"]
                sx, sy = L["strides"]
                nn.pulp_nn_conv_Ho_parallel(cur, None, P.get("bias"), out, P["w"], k, lam, mult, shift, W, H, Cc, Wo, Ho,
                                            Co, kx, ky, pt, pb, pl, pr, sx, sy, relu, bn)
            else:
                nn.pulp_nn_pointwise_HoWo_parallel(cur, None, P.get("bias"), out, P["w"], k, lam, mult, shift, W, H, Cc,
                                                   Wo, Ho, Co, 1, 1, 0, 0, 0, 0, 1, 1, relu, bn)
        elif op == "depthwise":
            k, lam, mult, shift, relu, bn = self._requant_args(L, P)
            ky, kx = L["w"].shape[1:3]
            pt, pb, pl, pr = L["pads"]
            sx, sy = L["strides"]
            fusable = (ky, kx) == (3, 3) and tuple(L["pads"]) == (1, 1, 1, 1) and sx == sy
            if self.fused and fusable and i not in self.unfused:
                try:
                    nn.depthwise_hwc(cur, P.get("bias"), out, P["w"], k, lam, mult, shift, W, H, Cc, Wo, Ho, sx, relu, bn)
                    return out
                except PulpNNError as err:
                    if err.code != 2:
                        raise
                    self.unfused.add(i)    # no fused kernel for this geometry
            chw = self.chw[L["name"]]
            nn.hwc_to_chw(cur, chw, W, H, Cc)
            nn.pulp_nn_depthwise_generic(chw, None, P.get("bias"), out, P["w"], None, k, lam, mult, shift, W, H, Cc,
                                         Wo, Ho, Cc, kx, ky, pt, pb, pl, pr, sx, sy, relu, bn)
        elif op == "maxpool":
            kx, ky = L["kernel"]
            sx, sy = L["strides"]
            pt, pb, pl, pr = L.get("pads", (0, 0, 0, 0))
            nn.pulp_nn_maxpool(cur, out, W, H, Cc, Wo, Ho, kx, ky, pt, pb, pl, pr, sx, sy)
        elif op == "avgpool":
            kx, ky = L["kernel"]
            sx, sy = L["strides"]
            pt, pb, pl, pr = L.get("pads", (0, 0, 0, 0))
            nn.pulp_nn_avgpool(cur, out, L.get("lam", 0), L.get("shift", 0), L.get("add", 0), W, H, Cc, Wo, Ho, kx, ky,
                               pt, pb, pl, pr, sx, sy, L.get("requant", 0))
        elif op == "linear":
            k, lam, mult, shift, relu, bn = self._requant_args(L, P)
            nn.pulp_nn_linear(cur, P.get("bias"), out, P["w"], k, lam, mult, shift, H * W * Cc, Co, relu, bn)
        elif op == "linear_out_32":
            nn.pulp_nn_linear_out_32(cur, P.get("bias"), out, P["w"], H * W * Cc, Co)
        else:
            raise ValueError(op)
        return out

    def run(self, x):
        """x: device tensor batch,H,W,C uint8.  Queues every layer; returns the last layer's tensor."""
        self.nn.set_batch(self.batch)
        tensors = {"input": x}
        out = x
        self.launches = 0
        i = 0
        while i < len(self.layers):
            L = self.layers[i]
            n = self._chain_length(i) if self.chain_blocks else 0
            if n >= 2 and self._queue_chain(i, n, tensors):
                last = self.layers[i + 2 * n - 1]["name"]
                out = tensors[last] = self.act[last]
                i += 2 * n
                continue
            if self._block_fusable(i) and self._queue_block(i, tensors):
                out = tensors[self.layers[i + 1]["name"]] = self.act[self.layers[i + 1]["name"]]
                i += 2
                continue
            out = tensors[L["name"]] = self._queue(i, tensors)
            self.launches += 2 if (L["op"] == "depthwise" and (not self.fused or i in self.unfused)) else 1
            i += 1
        return out

    # -- depthwise + pointwise as one launch ------------------------------------------------
    def _block_fusable(self, i, policy=True):
        """Layer i is a 3x3 / padding 1 depthwise layer whose only reader is the pointwise layer i + 1.
        policy=False: only whether the block can be one launch, not whether it pays on its own."""
        if not (self.fused and self.fuse_blocks) or i in self.unfused_blocks or i + 1 >= len(self.layers):
            return False
        L, N = self.layers[i], self.layers[i + 1]
        if L["op"] != "depthwise" or N["op"] != "pointwise" or N["in"] != L["name"]:
            return False
        # "auto": only where the single launch is not slower than the two.  Runner.tune() times both forms of every
        # such block on the batch at hand and records the faster one in block_choice.  Without that measurement the
        # rule is the shape of the fused kernel's work: it pays where an image's output plane is 8 x 8 pixels, so
        # that one workgroup takes whole images and each of its eight waves one item of the depthwise stage (on
        # MI355X at batch 256: 11.2 us against 5.9 + 6.4 for 16-pixel planes at stride 2, 11.8 against 5.4 + 7.1
        # for 8-pixel planes at stride 1); larger output planes split an image over workgroups that each run the
        # whole load -> depthwise -> MFMA -> store chain, smaller ones leave waves without an item.
        if policy and self.fuse_blocks == "auto":
            if i in self.block_choice:
                if not self.block_choice[i]:
                    return False
            elif tuple(self.shapes[L["name"]][:2]) != (8, 8):
                return False
        if L["op"] != "depthwise" or N["op"] != "pointwise" or N["in"] != L["name"]:
            return False
        sx, sy = L["strides"]
        if L["w"].shape[1:3] != (3, 3) or tuple(L["pads"]) != (1, 1, 1, 1) or sx != sy:
            return False
        readers = [M for M in self.layers if (M["in"] == L["name"] or (M["op"] == "add" and L["name"] in M["in"]))]
        return len(readers) == 1

    def _readers(self, name):
        return [M for M in self.layers if (M["in"] == name or (M["op"] == "add" and name in M["in"]))]

    def _chain_length(self, i):
        """How many depthwise + pointwise blocks of one shape start at layer i (stride 1, as many channels out as in,
        every intermediate tensor read by the next layer only): such a run is one launch, with the activations kept
        in LDS from block to block."""
        if i in self.unchained:
            return 0
        n, shape = 0, None
        while n < 8 and self._block_fusable(i + 2 * n, policy=False):
            L, N = self.layers[i + 2 * n], self.layers[i + 2 * n + 1]
            if L["strides"][0] != 1 or self.shapes[L["in"]] != self.shapes[N["name"]]:
                break
            if shape is None:
                shape = self.shapes[L["in"]]
            if self.shapes[L["in"]] != shape or (n > 0 and len(self._readers(L["in"])) != 1):
                break
            n += 1
        return n

    def _queue_chain(self, i, n, tensors):
        nn = self.nn
        H, W, Cc = self.shapes[self.layers[i]["in"]]
        blocks = []
        for j in range(n):
            L, P, N, Q = self.layers[i + 2 * j], self.params[i + 2 * j], self.layers[i + 2 * j + 1], self.params[i + 2 * j + 1]
            k1, l1, m1, s1, r1, b1 = self._requant_args(L, P)
            k2, l2, m2, s2, r2, b2 = self._requant_args(N, Q)
            blocks.append((P["w"], P.get("bias"), k1, l1, m1, s1, r1, b1, Q["w"], Q.get("bias"), k2, l2, m2, s2, r2, b2))
        try:
            nn.dw_pw_chain_hwc(tensors[self.layers[i]["in"]], self.act[self.layers[i + 2 * n - 1]["name"]], W, H, Cc, blocks)
        except PulpNNError as err:
            if err.code != 2:
                raise
            self.unchained.add(i)    # these blocks cannot share a launch
            return False
        self.launches += 1
        return True

    def _queue_block(self, i, tensors):
        L, P, N, Q, nn = self.layers[i], self.params[i], self.layers[i + 1], self.params[i + 1], self.nn
        H, W, Cc = self.shapes[L["in"]]
        Ho, Wo, Co = self.shapes[N["name"]]
        k1, l1, m1, s1, r1, b1 = self._requant_args(L, P)
        k2, l2, m2, s2, r2, b2 = self._requant_args(N, Q)
        try:
            nn.dw_pw_hwc(tensors[L["in"]], self.act[N["name"]], W, H, Cc, Wo, Ho, Co, L["strides"][0], P["w"], P.get("bias"),
                         k1, l1, m1, s1, r1, b1, Q["w"], Q.get("bias"), k2, l2, m2, s2, r2, b2)
        except PulpNNError as err:
            if err.code != 2:
                raise
            self.unfused_blocks.add(i)    # no fused kernel for this geometry
            return False
        self.launches += 1
        return True

    # -- calibration ------------------------------------------------------------------------
    def _calib_buffers(self):
        if self._calib is None:
            torch = self.torch
            most = max(self.batch * int(np.prod(self.shapes[L["name"]])) for L in self.layers)
            nbytes = self.nn.calib_workspace_bytes(most)
            self._calib = (torch.empty(nbytes // 8 + 1, dtype=torch.int64, device="cuda"), nbytes,
                           torch.zeros(2, dtype=torch.int64, device="cuda"))
        return self._calib

    def layer_absmax(self, i, tensors):
        """(max |acc * k|, derived out_shift) of conv-like layer i on the GPU."""
        L, P, nn = self.layers[i], self.params[i], self.nn
        ws, nbytes, res = self._calib_buffers()
        cur = tensors[L["in"]]
        H, W, Cc = self.shapes[L["in"]]
        Ho, Wo, Co = self.shapes[L["name"]]
        nn.set_batch(self.batch)
        if L["op"] == "depthwise":
            ky, kx = L["w"].shape[1:3]
            pt, _, pl, _ = L["pads"]
            sx, sy = L["strides"]
            nn.calib_depthwise(cur, P.get("bias"), P["w"], P["k"], W, H, Cc, Wo, Ho, kx, ky, pt, pl, sx, sy, 1, ws,
                               nbytes, res)
        elif L["op"] == "linear":
            nn.calib_conv(cur, P.get("bias"), P["w"], P["k"], 1, 1, H * W * Cc, 1, 1, Co, 1, 1, 0, 0, 1, 1, ws, nbytes, res)
        else:
            ky, kx = L["w"].shape[1:3]
            pt, _, pl, _ = L.get("pads", (0, 0, 0, 0))
            sx, sy = L.get("strides", (1, 1))
            nn.calib_conv(cur, P.get("bias"), P["w"], P["k"], W, H, Cc, Wo, Ho, Co, kx, ky, pt, pl, sx, sy, ws, nbytes, res)
        nn.sync()
        m, shift = (int(v) for v in res.cpu().numpy().view(np.uint64))
        if nn.bn_bits == 32 and m >= 2 ** 31:
            # the 32-bit tree forms acc * k in int32 (pulp_nn_utils.c:35-45): the layer's product wraps on this batch,
            # and no out_shift derived from the unwrapped maximum describes what the layer computes
            raise ValueError("layer %s: max |acc * k| = %d does not fit int32; the 32-bit batch-norm product wraps "
                             "(use smaller k or the 64-bit library)" % (L["name"], m))
        return m, shift

    def tune(self, x, reps=20):
        """Times every depthwise + pointwise block that can be one launch (and is not part of a chained run) both
        ways on this batch and keeps the faster form (fuse_blocks="auto" then follows these choices instead of the
        shape rule).  Needs every out_shift (run calibrate() first).  Returns {depthwise layer name: fused?}."""
        torch = self.torch
        self.nn.set_batch(self.batch)
        tensors = {"input": x}
        self.run(x)
        for L in self.layers:
            tensors[L["name"]] = self.act[L["name"]]
        self.nn.sync()

        def timed(fn):
            fn()
            self.nn.sync()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            self.nn.sync()
            return e0.elapsed_time(e1) / reps

        chosen = {}
        i = 0
        while i < len(self.layers):
            n = self._chain_length(i) if self.chain_blocks else 0
            if n >= 2:
                i += 2 * n
                continue
            if self._block_fusable(i, policy=False):
                ok = self._queue_block(i, tensors)   # False: the library has no fused kernel for this geometry
                if ok:
                    t_fused = timed(lambda: self._queue_block(i, tensors))
                    t_split = timed(lambda: (self._queue(i, tensors), self._queue(i + 1, tensors)))
                    self.block_choice[i] = t_fused <= t_split
                else:
                    self.block_choice[i] = False
                chosen[self.layers[i]["name"]] = self.block_choice[i]
                i += 2
                continue
            i += 1
        self.nn.sync()
        return chosen

    def calibrate(self, x, force=False):
        """Runs the chain on x and gives every batch-norm layer without an out_shift (all of them with
        force=True) the shift floor(log2(max |acc * k|)) - 7 measured on this batch.  Returns {name: shift}."""
        self.nn.set_batch(self.batch)
        tensors = {"input": x}
        chosen = {}
        for i, L in enumerate(self.layers):
            if L["op"] in CONV_LIKE and L.get("relu") and L.get("bn") and (force or L.get("shift") is None):
                _, L["shift"] = self.layer_absmax(i, tensors)
                chosen[L["name"]] = L["shift"]
            tensors[L["name"]] = self._queue(i, tensors)
        self.nn.sync()
        return chosen
