"""Host-side mirror of ``MyCaffe.extras/LlmInference.cs`` (:93-308): the wrapper the
C# host uses to drive the llama2 extension through ``CudaDnn.CreateExtension`` /
``RunExtension`` / ``RunExtensionEx`` / ``QueryExtensionStrings``.

Token-id generation (``GenerateIds`` / ``GenerateBatch``) has no counterpart in the
reference, whose only front door is a text prompt plus tokenizer file.
"""
import numpy as np

from .cudadnn import llama2_extension_path


class CUDAFN_EXTENSION_LLM:
    """CudaDnn.cs:22-52."""
    CREATE = 1
    DESTROY = 2
    LOAD = 3
    QUERY_STATUS = 4
    GENERATE = 5
    QUERY_RESPONSE = 6
    ABORT_GENERATE = 7
    GENERATE_IDS = 100
    SET_OPTION = 101
    GENERATE_BATCH = 102
    QUERY_TIMING = 103
    PROFILE_STEP = 104
    TOKENIZE = 105
    SAMPLE = 106
    RUNNING_SUM = 107


STEP_CLASSES = ("matvec_qkv", "rope_store", "attn_decode", "matvec_wo", "matvec_w13", "matvec_w2", "matvec_cls", "embed_argmax")


class LlmInference:
    def __init__(self, cuda):
        self.m_cuda = cuda
        self.m_hExtension = 0
        self.m_rgLlm = None

    def Initialize(self, strExtensionPath=None, fTemperature=0.0, fTopp=0.9, lSeed=0):
        """LlmInference.cs:93-125: CreateExtension, then CREATE {temperature, topp, seed}."""
        self.m_hExtension = self.m_cuda.CreateExtension(strExtensionPath or llama2_extension_path())
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.CREATE, [fTemperature, fTopp, lSeed])
        self.m_rgLlm = [float(rg[0])]

    def CleanUp(self):
        """LlmInference.cs:131-145."""
        if self.m_hExtension:
            if self.m_rgLlm is not None:
                self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.DESTROY, self.m_rgLlm)
                self.m_rgLlm = None
            self.m_cuda.FreeExtension(self.m_hExtension)
            self.m_hExtension = 0

    Dispose = CleanUp

    def SetOption(self, option, value):
        self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.SET_OPTION, self.m_rgLlm + [option, value])

    def Load(self, strModelFile, strTokenizerFile=""):
        """LlmInference.cs:150-190 (synchronous here): LOAD with "model;tokenizer"."""
        self.m_cuda.RunExtensionEx(self.m_hExtension, CUDAFN_EXTENSION_LLM.LOAD, self.m_rgLlm, strModelFile + ";" + strTokenizerFile)

    def QueryStatus(self):
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.QUERY_STATUS, self.m_rgLlm)
        return float(rg[0]), int(rg[1])

    def CancelGenerate(self):
        """LlmInference.cs:201-206."""
        self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.ABORT_GENERATE, self.m_rgLlm)

    def Generate(self, strPrompt):
        """LlmInference.cs:214-262: GENERATE with the rendered prompt text."""
        self.m_cuda.RunExtensionEx(self.m_hExtension, CUDAFN_EXTENSION_LLM.GENERATE, self.m_rgLlm, strPrompt)

    def QueryResponse(self):
        """LlmInference.cs:272-300: poll the response text; "\\n[END]" marks the end."""
        text = self.m_cuda.QueryExtensionStrings(self.m_hExtension, CUDAFN_EXTENSION_LLM.QUERY_RESPONSE, [int(self.m_rgLlm[0])])[0]
        end = text.endswith("\n[END]")
        return (text[:-6] if end else text), end

    def Tokenize(self, strText, bBos=True, bEos=False):
        """Token ids of ``strText`` from the tokenizer given at Load (addition of this library)."""
        rg = self.m_cuda.RunExtensionEx(self.m_hExtension, CUDAFN_EXTENSION_LLM.TOKENIZE, self.m_rgLlm + [int(bBos), int(bEos)], strText)
        return rg.astype(np.int32)

    def DecodePiece(self, nPrevToken, nToken):
        """The text piece a token contributes after ``nPrevToken`` (addition of this library)."""
        return self.m_cuda.QueryExtensionStrings(self.m_hExtension, CUDAFN_EXTENSION_LLM.TOKENIZE,
                                                 [int(self.m_rgLlm[0]), -1, int(nPrevToken), int(nToken)])[0]

    def Sample(self, logits):
        """One call of the handle's sampler on the given logits (advances its random state unless temperature is 0)."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.SAMPLE, self.m_rgLlm + [float(v) for v in logits])
        return int(rg[0])

    def RunningSum(self, values, threshold=float("inf")):
        """The device sampler's rounded running sum over non-negative fp32 ``values``: (first index at which the sum
        exceeds ``threshold`` or len(values), the sum reached as numpy.float32)."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.RUNNING_SUM,
                                      self.m_rgLlm + [float(threshold)] + [float(v) for v in values])
        return int(rg[0]), np.float32(rg[1])

    def GenerateIds(self, prompt_ids, nSteps, want_logits=False, vocab_size=None):
        """Greedy decode from token ids; returns the id sampled after every position
        (and, on request, every step's logits)."""
        args = self.m_rgLlm + [nSteps, 1 if want_logits else 0] + [float(t) for t in prompt_ids]
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.GENERATE_IDS, args)
        ids = rg[:nSteps].astype(np.int32)
        if want_logits:
            return ids, rg[nSteps:].reshape(nSteps, -1)
        return ids

    def GenerateBatch(self, prompts, nSteps, want_logits=False):
        """prompts: (batch, nPrompt) ids; returns (batch, nSteps) sampled ids (and, on request, the logits of
        every step, (batch, nSteps, vocabulary))."""
        p = np.asarray(prompts)
        args = self.m_rgLlm + [nSteps, p.shape[0], p.shape[1]] + [float(t) for t in p.reshape(-1)]
        self.SetOption(6, 1 if want_logits else 0)
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.GENERATE_BATCH, args)
        n = p.shape[0] * nSteps
        ids = rg[:n].astype(np.int32).reshape(p.shape[0], nSteps)
        if want_logits:
            return ids, rg[n:].reshape(p.shape[0], nSteps, -1)
        return ids

    def QueryTiming(self):
        """(milliseconds, steps) of the timed span of the last generation, from HIP events."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.QUERY_TIMING, self.m_rgLlm)
        return float(rg[0]), int(rg[1])

    def LastRunUsedGraph(self):
        """Whether the steps of the last generation were replays of the captured HIP graph (False: eager launches,
        either asked for with option 3 or because capture failed)."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.QUERY_TIMING, self.m_rgLlm)
        return bool(rg[2] != 0)

    def LastPrefill(self):
        """(milliseconds, rows) of the batched prompt pass of the last generation: HIP-event time on the engine's stream
        and sequences x prompt positions covered; (0, 0) when the prompt went one decode step per position."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.QUERY_TIMING, self.m_rgLlm)
        return float(rg[3]), int(rg[4])

    def ProfileStep(self, pos, reps=8, batch=1):
        """Per-kernel-class timing of eager decode steps at ``pos`` (HIP event pairs around
        every launch): {class: (ms per step, launches per step, algorithmic bytes per step)}, plus
        "_event_pair_ms": what such a pair measures around an empty kernel."""
        rg = self.m_cuda.RunExtension(self.m_hExtension, CUDAFN_EXTENSION_LLM.PROFILE_STEP, self.m_rgLlm + [pos, reps, batch])
        out = {name: (float(rg[3 * i]), float(rg[3 * i + 1]), float(rg[3 * i + 2])) for i, name in enumerate(STEP_CLASSES)}
        out["_event_pair_ms"] = float(rg[3 * len(STEP_CLASSES)])
        return out
