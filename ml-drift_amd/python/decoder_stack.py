"""The FullyConnected sequence of a decoder stack (Gemma-2B-like: hidden 2048, MQA k/v 256,
gated MLP 16384, int4 group-32 weights, fp16 tensors), as the reference's model builder emits
it per layer (samples/llm/gemma3_model_builder.cc:1115-1128): q, k, v, o, gate, up, down.

Only the FCs are reproduced (no attention, norm or activation): every FC reads a synthetic
N(0,1) activation tensor of its input width and writes its own output tensor, and the FCs run
in the graph's order on one stream, i.e. with the dependencies of the real layer.  Every FC of
every layer has weights and scales of its own (seed layer * 7 + index), so a decode step streams
the whole stack's 1.1 GB through HBM.  (What a GEMV or GEMM costs does not depend on the values of
its activations, so the synthetic inputs time like the fed-forward ones; the chain with the values
flowing through it is a parity test.)

Nothing here computes a result on the host.
"""
import numpy as np

import mldhip as M
import workloads as W


class DecoderStack:
    def __init__(self, layers=W.C5_LAYERS, max_tokens=128, seed=5, layer_shapes=None, device="cuda", keep_host=True,
                 decode_layout=False):
        import torch
        self.torch = torch
        self.layers = layers
        self.max_tokens = max_tokens
        self.shapes = list(layer_shapes or W.C5_LAYER)
        self.device = device
        # host-side cases: every FC of every layer has weights and scales of its own, seed
        # layer * 7 + index; the FCs of one input width share one synthetic N(0,1) activation tensor
        self.inputs = {}
        rng = np.random.default_rng(seed)
        for _, k, _ in self.shapes:
            if k not in self.inputs:
                self.inputs[k] = W.round_to(rng.standard_normal((max_tokens, k)), np.float16)
        self.keep_host = keep_host
        self.layer_cases = []
        self.tokens = None
        self.src = {}
        self.nodes = []  # (layer, case index, op, out tensor, weights, scales)
        self._weights = []
        for layer in range(layers):
            cases = []
            for idx, (name, k, n) in enumerate(self.shapes):
                case = W.make_fc_case(seed=layer * 7 + idx, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16,
                                      groups=k // 32)
                case["name"] = name
                case["m"] = max_tokens
                case["act"] = self.inputs[k]
                # decode_layout: the weights as a decode graph's ops ask for them (the prefill graph keeps
                # its own packed copy)
                desc, w = W.pack_fc_weights(case, decode_layout=decode_layout)
                sc = M.scale_to_tensor(case["scale"], M.FLOAT16).view(np.float16)
                w_dev = torch.from_numpy(w).to(device)
                s_dev = torch.from_numpy(sc).to(device)
                out = torch.zeros((W.div_up(n, 4), max_tokens, 4), dtype=torch.float16, device=device)
                op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, n, k, desc,
                                 scale_shape=(n, case["groups"]), max_tokens=max_tokens)
                self._weights.append((w_dev, s_dev))
                self.nodes.append((layer, idx, op, out, w_dev, s_dev))
                if not keep_host:  # the bench needs the shapes only
                    case = dict(case, w=None, scale=None)
                cases.append(case)
            self.layer_cases.append(cases)
        self.cases = self.layer_cases[0]
        self.set_tokens(1)

    def weight_bytes(self):
        """Packed weights + scales of the whole stack (the bytes a decode step must stream)."""
        return sum(w.numel() * w.element_size() + s.numel() * s.element_size() for w, s in self._weights)

    def flops(self, tokens):
        return self.layers * sum(2.0 * tokens * c["k"] * c["n"] for c in self.cases)

    def set_tokens(self, tokens):
        """Re-binds every FC for `tokens` tokens (the first `tokens` rows of the synthetic input)."""
        assert 1 <= tokens <= self.max_tokens
        torch = self.torch
        self.tokens = tokens
        self.src = {k: torch.from_numpy(W.to_slices(a[:tokens]).astype(np.float16)).to(self.device)
                    for k, a in self.inputs.items()}
        self.outs = []
        for layer, idx, op, out, w_dev, s_dev in self.nodes:
            case = self.cases[idx]
            view = out.view(-1)[: W.div_up(case["n"], 4) * tokens * 4].view(W.div_up(case["n"], 4), tokens, 4)
            op.bind([self.src[case["k"]], w_dev, s_dev], [view])
            op.set_shape(1, 1, tokens)
            self.outs.append(view)

    def launch(self, stream=None, fused=True):
        """One pass over the stack in node order.  With `fused`, the FCs of a layer that read the
        same tensor (q/k/v; gate/up) go out as one launch where the library can serve them
        together (decode), singly otherwise."""
        s = self.torch.cuda.current_stream().cuda_stream if stream is None else stream
        if not fused:
            for _, _, op, _, _, _ in self.nodes:
                op.launch(s)
            return
        names = [c["name"] for c in self.cases]
        per_layer = len(self.cases)
        groups = [[names.index(n) for n in grp] for grp in self.PARALLEL if all(n in names for n in grp)]
        for layer in range(self.layers):
            idx = 0
            while idx < per_layer:
                grp = next((g for g in groups if g[0] == idx and g == list(range(idx, idx + len(g)))), None)
                if grp is not None:
                    ops = [self.nodes[layer * per_layer + i][2] for i in grp]
                    try:
                        M.fc_launch_fused(ops, s)
                        idx += len(grp)
                        continue
                    except M.MldhipError as e:
                        if e.code != M.FAILED_PRECONDITION:
                            raise
                self.nodes[layer * per_layer + idx][2].launch(s)
                idx += 1

    # FCs of a layer that read the same tensor and do not depend on each other
    PARALLEL = (("q", "k", "v"), ("gate", "up"))

    def capture(self, parallel=False):
        """Captures one pass over the stack into a graph and returns it (replay with .replay()).
        With `parallel`, the FCs of a layer that are independent in the real graph (q/k/v; gate/up)
        are captured as parallel branches, each on its own stream of default priority; the
        dependent ones (o after q/k/v, down after gate/up, next layer after down) stay ordered.
        (On MI355X the fork/join of the branches costs more than the overlap gains: 1093 us
        against 873 us for a decode step, hence the default.)"""
        torch = self.torch
        self.launch(fused=False)  # warm-up
        torch.cuda.synchronize()
        main = torch.cuda.Stream()
        side = [torch.cuda.Stream(), torch.cuda.Stream()]
        names = [c["name"] for c in self.cases]
        group_of = {}
        for grp in self.PARALLEL:
            if parallel and all(n in names for n in grp):
                for n in grp:
                    group_of[n] = grp
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=main):
            per_layer = len(self.cases)
            for layer in range(self.layers):
                idx = 0
                while idx < per_layer:
                    name = names[idx]
                    grp = group_of.get(name)
                    if grp is None or name != grp[0]:
                        self.nodes[layer * per_layer + idx][2].launch(main.cuda_stream)
                        idx += 1
                        continue
                    fork = main.record_event()
                    members = [names.index(n) for n in grp]
                    self.nodes[layer * per_layer + members[0]][2].launch(main.cuda_stream)
                    for st, mi in zip(side, members[1:]):
                        st.wait_event(fork)
                        self.nodes[layer * per_layer + mi][2].launch(st.cuda_stream)
                        main.wait_event(st.record_event())
                    idx = max(members) + 1
        self._graph_streams = (main, side)
        return graph

    def result(self, layer, idx):
        self.torch.cuda.synchronize()
        pos = layer * len(self.cases) + idx
        return W.from_slices(self.outs[pos].cpu().numpy().astype(np.float32), self.cases[idx]["n"])

    def case(self, idx, tokens=None, layer=0):
        """The host-side case of FC `idx` of `layer` restricted to the current token count."""
        t = self.tokens if tokens is None else tokens
        c = dict(self.layer_cases[layer][idx])
        c["m"] = t
        c["act"] = c["act"][:t]
        return c

    def kernel_names(self):
        return [op.kernel_name for _, _, op, _, _, _ in self.nodes]
