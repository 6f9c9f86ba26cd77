"""Host mirror of the reference's RecurrentLayer (Prod/Layers/RecurrentLayer.cs) on GPUTensor.

The reference takes its SimpleRNN / LSTM / GRU layers from cuDNN; this class makes the same sequence of calls
against libsharpnet_hip.so: weight space and per-gate views (RecurrentLayer.cs:138-190), forward with the reserve
buffer kept for training (:305-408), backward data then backward weights into zeroed gradients (:410-520), with the
reference's handling of ``returnSequences == false`` (last step of the forward direction, first step of the reverse
one) and of the encoder / decoder pair: an encoder's output is its final hidden states followed by its final cell
states (two blocks of one buffer, RecurrentLayer.cs:526-533), a decoder takes that buffer as its initial states and
returns their gradients in the same arrangement.
"""
import ctypes

from .gpu_tensor import GPUTensor
from .hiplib import RnnDesc, check_status

# cudnnRNNMode_t / cudnnRNNBiasMode_t (Prod/GPU/CudnnWrapper.cs:313-327,396-410)
CUDNN_RNN_RELU, CUDNN_RNN_TANH, CUDNN_LSTM, CUDNN_GRU = range(4)
CUDNN_RNN_NO_BIAS, CUDNN_RNN_SINGLE_INP_BIAS, CUDNN_RNN_DOUBLE_BIAS, CUDNN_RNN_SINGLE_REC_BIAS = range(4)
_GATES = {CUDNN_RNN_RELU: 1, CUDNN_RNN_TANH: 1, CUDNN_LSTM: 4, CUDNN_GRU: 3}


class RecurrentLayer:
    def __init__(self, gpu_wrapper, inputSize, hiddenSize, cellMode, biasMode, returnSequences, isBidirectional,
                 numLayers=1, isEncoderThatWillBeFollowedByDecoder=False, dropoutRate=0.0):
        if isEncoderThatWillBeFollowedByDecoder and returnSequences:
            raise ValueError("an Encoder can not return a sequence")            # RecurrentLayer.cs:128-131
        if isEncoderThatWillBeFollowedByDecoder and numLayers != 1:
            # The context vector is two (batch, K*hidden) blocks, the library's states are (K*layers, batch, hidden):
            # with more than one layer they do not have the same size and the state pointers would run past the buffer.
            raise ValueError("an Encoder followed by a Decoder must have exactly one layer")
        self.IsEncoderThatWillBeFollowedByDecoder = isEncoderThatWillBeFollowedByDecoder
        self.Wrapper = gpu_wrapper
        self._lib = gpu_wrapper.lib
        self.desc = RnnDesc(cell_mode=cellMode, bias_mode=biasMode, bidirectional=bool(isBidirectional),
                            num_layers=numLayers, input_size=inputSize, hidden_size=hiddenSize,
                            dropout=dropoutRate)                                 # RecurrentLayer.cs:69,123
        self._returnSequences = returnSequences
        self.hidden_size, self.input_size, self.num_layers = hiddenSize, inputSize, numLayers
        self.K = 2 if isBidirectional else 1
        nbytes = ctypes.c_size_t()
        check_status(self._lib.snhip_rnn_weight_space_size(ctypes.byref(self.desc), ctypes.byref(nbytes)),
                     "snhip_rnn_weight_space_size")
        self._weightsAndBiases = GPUTensor([nbytes.value // 4], None, gpu_wrapper)
        self._weightsAndBiasesGradients = GPUTensor([nbytes.value // 4], None, gpu_wrapper)
        self._weightsAndBiases.ZeroMemory()
        self._weightsAndBiasesGradients.ZeroMemory()
        # the per-gate views of RecurrentLayer.cs:164-190
        self._weight_ih, self._weight_hh, self._bias_ih, self._bias_hh = [], [], [], []
        self._weight_ih_gradients, self._weight_hh_gradients, self._bias_ih_gradients, self._bias_hh_gradients = [], [], [], []
        G = _GATES[cellMode]
        for pseudoLayer in range(self.K * numLayers):
            for linLayerID in range(2 * G):
                off, rows, cols, boff = ctypes.c_longlong(), ctypes.c_int(), ctypes.c_int(), ctypes.c_longlong()
                check_status(self._lib.snhip_rnn_weight_params(ctypes.byref(self.desc), pseudoLayer, linLayerID,
                                                               ctypes.byref(off), ctypes.byref(rows), ctypes.byref(cols),
                                                               ctypes.byref(boff)), "snhip_rnn_weight_params")
                isAx = linLayerID < G
                for space, wl, bl in ((self._weightsAndBiases, self._weight_ih if isAx else self._weight_hh,
                                       self._bias_ih if isAx else self._bias_hh),
                                      (self._weightsAndBiasesGradients,
                                       self._weight_ih_gradients if isAx else self._weight_hh_gradients,
                                       self._bias_ih_gradients if isAx else self._bias_hh_gradients)):
                    wl.append(space.Slice(off.value, [rows.value, cols.value]))
                    bl.append(space.Slice(boff.value, [rows.value]) if boff.value >= 0 else None)
        self._reserveSpace = None
        self._workSpace = None
        self._yIfReturnSequences = None

    def Dispose(self):
        for t in (self._weightsAndBiases, self._weightsAndBiasesGradients, self._reserveSpace, self._workSpace,
                  self._yIfReturnSequences):
            if t is not None and t.IsOwnerOfMemory:
                t.Dispose()

    def OutputShape(self, batchSize, timeSteps):
        # RNNDescriptor.Y_Shape (Prod/Layers/RNNDescriptor.cs:49-60): an encoder returns hidden and cell states
        K = self.K * (2 if self.IsEncoderThatWillBeFollowedByDecoder else 1)
        if self._returnSequences:
            return [batchSize, timeSteps, K * self.hidden_size]
        return [batchSize, K * self.hidden_size]

    @staticmethod
    def _ExtractEncoderContextVector(t):
        """(hidden states, cell states): the two halves of an encoder's output buffer (RecurrentLayer.cs:526-533)."""
        shape = list(t.Shape)
        shape[-1] //= 2
        return t.Slice(0, shape), t.Slice(t.Count // 2, shape)

    def _CheckDecoderArguments(self, contextVector, batchSize):
        """A context vector (an encoder's output or its gradient) holds K*batch*hidden floats per block, which is what
        the library reads and writes as initial states only when this layer has one layer: refuse anything else
        instead of letting the device run past the buffer."""
        if contextVector is None:
            return
        if self.num_layers != 1:
            raise ValueError("a Decoder that takes an encoder's output must have exactly one layer (has %d)" % self.num_layers)
        if contextVector.Count != 2 * self.K * batchSize * self.hidden_size:
            raise ValueError("encoder output has %d elements, expected 2 x %d x %d x %d"
                             % (contextVector.Count, self.K, batchSize, self.hidden_size))

    def _buffers(self, isTraining, batchSize, timeSteps):
        ws, rs = ctypes.c_size_t(), ctypes.c_size_t()
        check_status(self._lib.snhip_rnn_temp_space_sizes(ctypes.byref(self.desc), int(isTraining), batchSize, timeSteps,
                                                          ctypes.byref(ws), ctypes.byref(rs)), "snhip_rnn_temp_space_sizes")
        return ws.value, rs.value

    def ForwardPropagation(self, x, yFull, isTraining, encoderOutput=None):
        """x (batch, steps, input); yFull (batch, steps, K*hidden) or (batch, K*hidden), twice as wide for an encoder;
        encoderOutput: the output of the encoder this layer decodes (RecurrentLayer.cs:305-408)."""
        batchSize, timeSteps = x.Shape[0], x.Shape[1]
        assert x.Shape[2] == self.input_size and yFull.Shape == self.OutputShape(batchSize, timeSteps)
        self._CheckDecoderArguments(encoderOutput, batchSize)
        y, cy = self._ExtractEncoderContextVector(yFull) if self.IsEncoderThatWillBeFollowedByDecoder else (yFull, None)
        hx, cx = self._ExtractEncoderContextVector(encoderOutput) if encoderOutput is not None else (None, None)
        ws_bytes, rs_bytes = self._buffers(isTraining, batchSize, timeSteps)
        workSpace = GPUTensor([ws_bytes // 4], None, self.Wrapper)
        self._reserveSpace = GPUTensor([rs_bytes // 4], None, self.Wrapper) if isTraining else None
        if self._returnSequences:
            ySeq, hy = y, None
        else:
            ySeq = GPUTensor([batchSize, timeSteps, self.K * self.hidden_size], None, self.Wrapper)
            # hy (K, batch, hidden) of the top layer; the lower layers' final states go to a scratch tensor
            hyAll = GPUTensor([self.K * self.num_layers, batchSize, self.hidden_size], None, self.Wrapper)
            hy = hyAll
        cyAll = GPUTensor([self.K * self.num_layers, batchSize, self.hidden_size], None, self.Wrapper) if cy is not None else None
        check_status(self._lib.snhip_rnn_forward(
            self.Wrapper.handle, ctypes.byref(self.desc), int(isTraining), batchSize, timeSteps, x.Pointer, ySeq.Pointer,
            hx.Pointer if hx is not None else None, hy.Pointer if hy is not None else None,
            cx.Pointer if cx is not None else None, cyAll.Pointer if cyAll is not None else None,
            self._weightsAndBiases.Pointer, workSpace.Pointer, ws_bytes,
            self._reserveSpace.Pointer if isTraining else None, rs_bytes), "snhip_rnn_forward")
        if not self._returnSequences:
            top = hyAll.Slice((self.num_layers - 1) * self.K * batchSize * self.hidden_size,
                              [self.K, batchSize, self.hidden_size])
            if self.K == 2:
                # (K, batch, hidden) -> (batch, K*hidden): Switch_First_2_axis, RecurrentLayer.cs:376-391
                top.Reshape(1, self.K, batchSize, self.hidden_size).TransposeSecondAndThirdDimension(
                    y.Reshape(1, batchSize, self.K, self.hidden_size))
            else:
                top.CopyTo(y)
            if cyAll is not None:             # the top layer's cell states, (K, batch, hidden) as cuDNN leaves them
                cyAll.Slice((self.num_layers - 1) * self.K * batchSize * self.hidden_size,
                            [self.K, batchSize, self.hidden_size]).CopyTo(cy)
                cyAll.Dispose()
            hyAll.Dispose()
            if isTraining:
                self._yIfReturnSequences = ySeq
            else:
                ySeq.Dispose()
        workSpace.Dispose()

    def BackwardPropagation(self, x, yFull, dyFull, dx, encoderOutput=None, dEncoderOutput=None):
        """RecurrentLayer.cs:410-520.  dx may be None (previous layer is the input).  A decoder also takes the encoder's
        output again and writes the gradient with respect to it (hidden block, cell block) into dEncoderOutput."""
        assert self._reserveSpace is not None
        batchSize, timeSteps = x.Shape[0], x.Shape[1]
        H, K = self.hidden_size, self.K
        self._CheckDecoderArguments(encoderOutput, batchSize)
        self._CheckDecoderArguments(dEncoderOutput, batchSize)
        y, _ = self._ExtractEncoderContextVector(yFull) if self.IsEncoderThatWillBeFollowedByDecoder else (yFull, None)
        dy, dcy = self._ExtractEncoderContextVector(dyFull) if self.IsEncoderThatWillBeFollowedByDecoder else (dyFull, None)
        hx, cx = self._ExtractEncoderContextVector(encoderOutput) if encoderOutput is not None else (None, None)
        dhx, dcx = self._ExtractEncoderContextVector(dEncoderOutput) if dEncoderOutput is not None else (None, None)
        if self._returnSequences:
            ySeq, dySeq = y, dy
        else:
            ySeq = self._yIfReturnSequences
            dySeq = GPUTensor(ySeq.Shape, None, self.Wrapper)
            dySeq.ZeroMemory()
            # last step takes the first half of dy, the first step (reverse direction) the second half (:437-454)
            for batchId in range(batchSize):
                dy.Slice(batchId * K * H, [H]).CopyTo(dySeq.Slice((batchId * timeSteps + timeSteps - 1) * K * H, [H]))
                if K == 2:
                    dy.Slice(batchId * K * H + H, [H]).CopyTo(dySeq.Slice(batchId * timeSteps * K * H + H, [H]))
        ws_bytes, rs_bytes = self._buffers(True, batchSize, timeSteps)
        workSpace = GPUTensor([ws_bytes // 4], None, self.Wrapper)
        ptr = lambda t: t.Pointer if t is not None else None
        # cell-state gradients travel as (K * layers, batch, hidden); with one layer that is the block itself
        dcyAll = None
        if dcy is not None:
            dcyAll = GPUTensor([K * self.num_layers, batchSize, H], None, self.Wrapper)
            dcyAll.ZeroMemory()
            dcy.CopyTo(dcyAll.Slice((self.num_layers - 1) * K * batchSize * H, [K, batchSize, H]))
        check_status(self._lib.snhip_rnn_backward_data(
            self.Wrapper.handle, ctypes.byref(self.desc), batchSize, timeSteps, ySeq.Pointer, dySeq.Pointer,
            ptr(dx), ptr(hx), None, ptr(dhx), ptr(cx), ptr(dcyAll), ptr(dcx), self._weightsAndBiases.Pointer,
            workSpace.Pointer, ws_bytes, self._reserveSpace.Pointer, rs_bytes), "snhip_rnn_backward_data")
        self._weightsAndBiasesGradients.ZeroMemory()
        check_status(self._lib.snhip_rnn_backward_weights(
            self.Wrapper.handle, ctypes.byref(self.desc), batchSize, timeSteps, x.Pointer, ptr(hx), ySeq.Pointer,
            self._weightsAndBiasesGradients.Pointer, workSpace.Pointer, ws_bytes, self._reserveSpace.Pointer, rs_bytes),
            "snhip_rnn_backward_weights")
        workSpace.Dispose()
        if dcyAll is not None:
            dcyAll.Dispose()
        self._reserveSpace.Dispose()
        self._reserveSpace = None
        if not self._returnSequences:
            dySeq.Dispose()
            self._yIfReturnSequences.Dispose()
            self._yIfReturnSequences = None
