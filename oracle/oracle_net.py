"""Net-level CPU oracle: the reference's layer builders, per-batch forward pass and
training step restated over the C oracle.  TEST INFRASTRUCTURE ONLY.

Builders follow SparseConvNetCUDA.cu:50-111 (addLearntLayer rounding to 32,
filterSize 1 adds no gather layer, poolSize 1 adds no pooling layer),
:165-196 (triangular builders, including the argument mix-up that makes the
convolution's minActiveInputs equal to the pool size) and :198-210 (spatial
sizes worked out from the top).  forward() follows BatchProducer.cu:40-87
(every layer's preprocess) and SparseConvNetCUDA.cu:227-247 (forwards loop,
then SoftmaxClassifier); train_step() follows :247-252 and every layer's
backwards().  What the reference draws from its clock-seeded RNG (dropout
subsets, fractional max-pooling regions) is an argument here: parity unpinned
for the draw itself, pinned for everything computed from it.
"""
import numpy as np

import oracle as orc

RELU, SOFTMAX, PRELU = orc.RELU, orc.SOFTMAX, orc.PRELU


def int_round(a, d):  # utilities.cu:103
    return int(np.floor(a * 1.0 / d + 0.5)) * d if a >= 0 else -int(np.floor(-a * 1.0 / d + 0.5)) * d


class Net:
    def __init__(self, dimension, nInputFeatures, nClasses, nTop=1, triangular=False):
        self.dimension, self.nInputFeatures, self.nClasses, self.nTop = dimension, nInputFeatures, nClasses, nTop
        self.triangular = triangular
        self.nOutputFeatures = nInputFeatures
        self.layers = []  # dicts: kind, geometry, nIn, nOut, act, dropout
        self.weights = {}
        self.inputSpatialSize = None

    # ---- builders
    def _learnt(self, nFeatures, act, dropout):
        if act != SOFTMAX:
            nFeatures = max(32, int_round(nFeatures, 32))
        if dropout > 0:
            kept = int(np.float32(nFeatures) * (np.float32(1) - np.float32(dropout)))  # float -> int argument
            dropout = np.float32(1) - (np.float32(int_round(kept, 32)) + np.float32(0.01)) * np.float32(1.0) / np.float32(nFeatures)
        dropout = max(float(dropout), 0.0)
        kind = "nin_prelu" if act == PRELU else "nin"
        self.layers.append(dict(kind=kind, nIn=self.nOutputFeatures, nOut=nFeatures, act=act, dropout=dropout))
        self.nOutputFeatures = nFeatures

    def addLeNetLayerMP(self, nFeatures, filterSize, filterStride, poolSize, poolStride, activationFn=RELU, dropout=0.0,
                        minActiveInputs=1):
        tri = self.triangular
        if tri:
            minActiveInputs = poolSize  # SparseConvNetCUDA.cu:165-168 vs :183-185
        if filterSize > 1:
            fs = orc.lib.orc_triangle_size(filterSize, self.dimension) if tri else filterSize ** self.dimension
            self.layers.append(dict(kind="conv_tri" if tri else "conv", size=filterSize, stride=filterStride,
                                    minActive=minActiveInputs, nIn=self.nOutputFeatures,
                                    nOut=self.nOutputFeatures * fs, fs=fs))
            self.nOutputFeatures *= fs
        self._learnt(nFeatures, activationFn, dropout)
        if poolSize > 1:
            self.layers.append(dict(kind="maxpool_tri" if tri else "maxpool", size=poolSize, stride=poolStride, nIn=0, nOut=0))

    def addLeNetLayerFMP(self, kind, nFeatures, filterSize, filterStride, poolSize, fmpShrink, activationFn=RELU,
                         dropout=0.0, minActiveInputs=1):
        """addLeNetLayerPOFMP / PDFMP / ROFMP / RDFMP (kind 0..3), SparseConvNetCUDA.cu:112-163"""
        assert not self.triangular
        if filterSize > 1:
            fs = filterSize ** self.dimension
            self.layers.append(dict(kind="conv", size=filterSize, stride=filterStride, minActive=minActiveInputs,
                                    nIn=self.nOutputFeatures, nOut=self.nOutputFeatures * fs, fs=fs))
            self.nOutputFeatures *= fs
        self._learnt(nFeatures, activationFn, dropout)
        if fmpShrink > 1:
            self.layers.append(dict(kind="fmp", fmpKind=kind, size=poolSize, shrink=np.float32(fmpShrink), nIn=0, nOut=0))

    def addTerminalPoolingLayer(self, poolSize):
        self.layers.append(dict(kind="terminal", size=poolSize, nIn=0, nOut=0))

    def _sizes_from(self, top):
        s = top
        for l in reversed(self.layers):
            l["outSize"] = s
            if l["kind"] in ("conv", "conv_tri", "maxpool", "maxpool_tri"):
                s = l["size"] + (s - 1) * l["stride"]
            elif l["kind"] == "fmp":  # MaxPoolingLayer.cu:211-217: float product, + 0.5 in double, truncated
                t = int(np.float64(np.float32(s) * l["shrink"]) + 0.5)
                s = t + 1 if t == s else t
            elif l["kind"] == "terminal":
                assert s == 1
                s = l["size"]
            l["inSize"] = s
        self.inputSpatialSize = s
        return s

    def addSoftmaxLayer(self):
        self._learnt(self.nClasses, SOFTMAX, 0.0)
        self._sizes_from(1)

    def finishHeadless(self, topSpatialSize):
        return self._sizes_from(topSpatialSize)

    def layer_list(self):
        return [dict(kind=l["kind"], nIn=l.get("nIn", 0) if l["kind"] in ("conv", "conv_tri", "nin", "nin_prelu") else 0,
                     nOut=l.get("nOut", 0) if l["kind"] in ("conv", "conv_tri", "nin", "nin_prelu") else 0,
                     act=l.get("act", -1) if l["kind"] in ("nin", "nin_prelu") else -1) for l in self.layers]

    def set_weights(self, layer, W, B, prelu=None):
        self.weights[layer] = (np.asarray(W, np.float32), np.asarray(B, np.float32),
                               None if prelu is None else np.asarray(prelu, np.float32))

    # ---- forward over one batch
    def forward(self, batch, sample, key, row, bg, features, nSpatialSites, labels=None, keep=True, ticks=None,
                present=None, rescale=False):
        """Returns a list of interfaces (dicts with grids, rules, features,
        choices, nSpatialSites, nFeatures, spatialSize) and, when the net ends
        in the classifier, probabilities / predictions / mistakes / nll.
        ticks: {layer index: (inputL, inputR)} for fractional max-pooling layers (the random draw is the caller's).
        present: a TRAINBATCH with dropout -- {NiN layer index: the output features kept} (again the caller's draw);
        feature matrices then hold the kept columns only (featuresPresent of the reference).
        rescale: a RESCALEBATCH -- no dropout scaling, and every NiN layer's weights are rescaled right after its
        forward pass (SparseConvNetCUDA.cu:230-241, NetworkInNetworkLayer.cu:203-218); self.weights changes."""
        scalingUnderneath = np.float32(1)
        d = self.dimension
        g = orc.Grids.from_flat(batch, sample, key, row, bg)
        feats = np.ascontiguousarray(features, np.float32)
        ifaces = [dict(grids=g, rules=np.zeros(0, np.int32), features=feats, choices=np.zeros(0, np.int32),
                       nSpatialSites=nSpatialSites, nFeatures=self.nInputFeatures, spatialSize=self.inputSpatialSize,
                       present=np.arange(self.nInputFeatures))]
        for i, l in enumerate(self.layers):
            k = l["kind"]
            cur = ifaces[-1]
            nxt = dict(grids=cur["grids"], rules=np.zeros(0, np.int32), choices=np.zeros(0, np.int32),
                       nFeatures=cur["nFeatures"], spatialSize=cur["spatialSize"], nSpatialSites=cur["nSpatialSites"],
                       present=cur["present"])
            width = len(cur["present"])  # columns of the input's feature matrix
            if k in ("conv", "conv_tri", "maxpool", "maxpool_tri"):
                fn = orc.rules_triangular if k.endswith("_tri") else orc.rules_square
                minActive = l.get("minActive", 1)
                og, rules, n = fn(cur["grids"], d, l["inSize"], l["outSize"], l["size"], l["stride"], minActive)
                nxt.update(grids=og, rules=rules, nSpatialSites=n, spatialSize=l["outSize"])
                if k.startswith("conv"):
                    nxt["features"] = orc.gather_rows(cur["features"], rules, width).reshape(n, -1)
                    nxt["nFeatures"] = cur["nFeatures"] * l["fs"]
                    # convolutionFeaturesPresent, ConvolutionalLayer.cu:74-80
                    nxt["present"] = np.concatenate([cur["present"] + cur["nFeatures"] * q for q in range(l["fs"])])
                else:
                    ps = rules.size // max(n, 1)
                    nxt["features"], ch = orc.maxpool(cur["features"], rules, n, ps, width)
                    nxt["choices"] = ch.reshape(-1)
            elif k == "fmp":
                inL, inR = ticks[i]
                og, rules, n = orc.rules_fmp(cur["grids"], d, l["inSize"], l["outSize"], l["size"], inL, inR,
                                             l["fmpKind"] in (0, 2))
                nxt.update(grids=og, rules=rules, nSpatialSites=n, spatialSize=l["outSize"])
                ps = rules.size // max(n, 1)
                nxt["features"], ch = orc.maxpool(cur["features"], rules, n, ps, width)
                nxt["choices"] = ch.reshape(-1)
            elif k in ("nin", "nin_prelu"):
                W, B, pr = self.weights[i]
                inP = cur["present"]
                outP = np.asarray(present[i]) if present is not None and i in present else np.arange(l["nOut"])
                nxt["present"] = outP
                if present is not None and len(inP) + len(outP) < l["nIn"] + l["nOut"]:
                    # the training branch, NetworkInNetworkLayer.cu:162-184: sub-matrix, no scaling
                    assert pr is None or len(outP) == l["nOut"]
                    w = np.ascontiguousarray(W[np.ix_(inP, outP)])
                    nxt["features"] = orc.nin_forward(cur["features"], w, B[outP], pr, 1.0, l["act"])
                    nxt["shrunk"] = (inP, outP, w)
                else:
                    p = np.float32(1.0) - (np.float32(0) if rescale else np.float32(l["dropout"]))
                    nxt["features"] = orc.nin_forward(cur["features"], W, B, pr, p, l["act"])
                nxt["nFeatures"] = l["nOut"]
                if rescale:
                    scale = np.float32(np.abs(nxt["features"].astype(np.float64)).sum() / nxt["features"].size)
                    nxt["featureScale"] = scale
                    scale = np.float32(1) if i == len(self.layers) - 1 else np.float32(np.power(scale, np.float32(-0.1)))
                    MW, MB, MP = getattr(self, "momentum", {}).get(i, (None, None, None))
                    self.weights[i] = (W * (scale / scalingUnderneath), B * scale, pr)
                    if MW is not None:
                        self.momentum[i] = (MW * (scale / scalingUnderneath), MB * scale, MP)
                    scalingUnderneath = scale
            elif k == "terminal":
                og, rules, S = orc.rules_terminal(cur["grids"])
                nxt.update(grids=og, rules=rules, nSpatialSites=batch, spatialSize=1)
                nxt["features"] = orc.terminal_pool(cur["features"], rules, batch, S, width)
            if not keep:
                cur.pop("features", None)
            ifaces.append(nxt)
        out = dict(interfaces=ifaces)
        if self.layers and self.layers[-1].get("act") == SOFTMAX:
            probs = ifaces[-1]["features"]
            out["probabilities"] = probs
            if labels is not None:
                pred, mistakes, nll = orc.softmax_classifier(probs, labels, self.nTop)
                out.update(predictions=pred, mistakes=mistakes, nll=nll)
            else:
                out["predictions"] = np.stack([orc.top_indices(p, self.nTop) for p in probs])
        return out

    # ---- the same pass in float64, through rule books that forward() has built
    def forward64(self, fwd, every=False):
        """Class probabilities (or the top feature matrix of a headless stack) of the batch behind `fwd` in float64
        numpy arithmetic: the rule books are taken from fwd's interfaces, every feature layer is evaluated from its
        definition (gather = indexing through the rules, NiN = p (A W + B) then the activation, max-pool = maximum
        of the listed rows, terminal pooling = mean of the listed rows).  Shares no arithmetic with the C oracle; it is
        what single-precision results are measured against.  Dropout subsets are taken from fwd; a RESCALEBATCH pass is not covered.
        every: an iterator over all interfaces' feature matrices instead, the input first (one alive at a time)."""
        it = self._forward64(fwd)
        if every:
            return it
        x = None
        for x in it:
            pass
        return x

    def _forward64(self, fwd):
        ifaces = fwd["interfaces"]
        x = ifaces[0]["features"].astype(np.float64).reshape(ifaces[0]["nSpatialSites"], -1)
        yield x
        for i, l in enumerate(self.layers):
            k, nxt = l["kind"], ifaces[i + 1]
            n = nxt["nSpatialSites"]
            if k in ("conv", "conv_tri"):
                r = nxt["rules"].reshape(n, -1)
                x = np.where((r >= 0)[:, :, None], x[np.maximum(r, 0)], 0.0).reshape(n, -1)
            elif k in ("maxpool", "maxpool_tri", "fmp"):
                r = nxt["rules"].reshape(n, -1)
                cand = np.where((r >= 0)[:, :, None], x[np.maximum(r, 0)], -np.inf)
                x = cand.max(1)
            elif k in ("nin", "nin_prelu"):
                W, B, pr = self.weights[i]
                if "shrunk" in nxt:  # a training batch with dropout: the sub-matrix, unscaled
                    _, outP, w = nxt["shrunk"]
                    z = x @ w.astype(np.float64) + B[outP].astype(np.float64)
                else:
                    p = 1.0 - float(np.float32(l["dropout"]))
                    z = p * (x @ W.astype(np.float64) + B.astype(np.float64))
                act = l["act"]
                if act == SOFTMAX:  # SigmoidLayer.cu:160-177
                    e = np.exp(z - np.maximum(z.max(1, keepdims=True), -10000.0))
                    x = e / e.sum(1, keepdims=True)
                elif act == orc.TANH:
                    x = np.tanh(z)
                elif act == orc.SIGMOID:
                    x = 1.0 / (1.0 + np.exp(-z))
                elif act == orc.NOSIGMOID:
                    x = z
                else:
                    slope = {RELU: 0.0, orc.VLEAKYRELU: float(np.float32(0.333)),
                             orc.LEAKYRELU: float(np.float32(0.01))}.get(act)
                    slope = pr.astype(np.float64) if act == PRELU else slope
                    x = np.where(z > 0, z, z * slope)
            elif k == "terminal":
                r = nxt["rules"].reshape(n, -1)
                cnt = np.maximum((r >= 0).sum(1), 1)
                x = np.where((r >= 0)[:, :, None], x[np.maximum(r, 0)], 0.0).sum(1) / cnt[:, None]
            yield x

    # ---- backward over the batch just forwarded, and the weight update
    def train_step(self, fwd, labels, learningRate, momentum):
        """SparseConvNetCUDA::processBatch for a TRAINBATCH without dropout (SparseConvNetCUDA.cu:247-252):
        SoftmaxClassifier's gradient, then backwards() of every layer, last to first.  Leaves the gradient of each
        interface in its dict ("dfeatures", where the reference computes one) and updates self.weights and
        self.momentum in place."""
        ifaces = fwd["interfaces"]
        if not hasattr(self, "momentum"):
            self.momentum = {}
        backprop = [False]
        for l in self.layers:  # output.backpropErrors of every layer's preprocess()
            backprop.append(True if l["kind"] in ("nin", "nin_prelu") else backprop[-1])
        ifaces[-1]["dfeatures"] = orc.softmax_grad(ifaces[-1]["features"], labels)
        for i in range(len(self.layers) - 1, -1, -1):
            l, cur, nxt = self.layers[i], ifaces[i], ifaces[i + 1]
            k = l["kind"]
            if k in ("nin", "nin_prelu"):
                W, B, pr = self.weights[i]
                W, B = W.copy(), B.copy()
                pr = None if pr is None else pr.copy()
                MW, MB, MP = self.momentum.get(i, (np.zeros_like(W), np.zeros_like(B),
                                                   None if pr is None else np.zeros_like(pr)))
                dZ, dB, dPr = orc.activation_backward(nxt["features"], nxt["dfeatures"], l["act"], pr)
                nxt["dfeatures"] = dZ  # in place in the reference
                if pr is not None:
                    orc.nag_update(dPr, MP, pr, learningRate, momentum, keepPositive=True)
                dW = orc.sgemm_AtB(cur["features"], dZ)
                if "shrunk" in nxt:  # NetworkInNetworkLayer.cu:235-263: only the entries the batch used move
                    inP, outP, w = nxt["shrunk"]
                    if backprop[i]:
                        cur["dfeatures"] = orc.sgemm_ABt(dZ, w)
                    ix = np.ix_(inP, outP)
                    subW, subM = np.ascontiguousarray(W[ix]), np.ascontiguousarray(MW[ix])
                    orc.nag_update(dW, subM, subW, learningRate, momentum)
                    W[ix], MW[ix] = subW, subM
                    subB, subMB = np.ascontiguousarray(B[outP]), np.ascontiguousarray(MB[outP])
                    orc.nag_update(dB, subMB, subB, learningRate, momentum)
                    B[outP], MB[outP] = subB, subMB
                else:
                    if backprop[i]:
                        cur["dfeatures"] = orc.sgemm_ABt(dZ, W)
                    orc.nag_update(dW, MW, W, learningRate, momentum)
                    orc.nag_update(dB, MB, B, learningRate, momentum)
                self.weights[i] = (W, B, pr)
                self.momentum[i] = (MW, MB, MP)
                nxt["dW"], nxt["dB"], nxt["dPReLU"] = dW, dB, dPr
            elif not backprop[i]:
                continue
            elif k in ("conv", "conv_tri"):
                width = len(cur["present"])
                cur["dfeatures"] = orc.gather_rows_backward(nxt["dfeatures"].reshape(-1, width), nxt["rules"],
                                                            cur["nSpatialSites"], width)
            elif k in ("maxpool", "maxpool_tri", "fmp"):
                cur["dfeatures"] = orc.maxpool_backward(nxt["dfeatures"], nxt["choices"], cur["nSpatialSites"])
            elif k == "terminal":
                S = nxt["rules"].size // max(nxt["nSpatialSites"], 1)
                cur["dfeatures"] = orc.terminal_pool_backward(nxt["dfeatures"], nxt["rules"], S, cur["nSpatialSites"])
        return fwd
