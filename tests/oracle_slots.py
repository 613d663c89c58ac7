"""CPU restatement of the reference's FP8 slot state machines over the oracle's primitives.

ActSlotOracle follows fp8_quant_act (src/trainer.cu:4732-4851) branch by branch with the slot fields of
src/trainer.cu:3247-3279 and the initial values of alloc_act_slot (src/trainer.cu:4176-4201).  Test infrastructure.
"""
import numpy as np

import oracle_lib as orc

E4M3_MAX, E5M2_MAX = np.float32(448.0), np.float32(57344.0)


class ActSlotOracle:
    def __init__(self, history_len=8, fp8_max=E4M3_MAX, calib_calls=8, spread_threshold=4.0):
        self.fp8_max = np.float32(fp8_max)
        self.delayed = orc.DelayedState(history_len)
        self.amax = np.float32(0)
        self.scale_snapshot = np.float32(0)
        self.descale_snapshot = np.float32(0)
        self.init = False
        self.calib_remaining = calib_calls
        self.calib_commit_pending = False
        self.calib_min = np.array([0x7f7f7f7f], np.uint32).view(np.float32)[0]      # src/trainer.cu:4197
        self.calib_max = np.float32(0)
        self.spread_threshold = np.float32(spread_threshold)

    @property
    def scale(self):
        return self.delayed.scale[0]

    @property
    def descale(self):
        return self.delayed.descale[0]

    def is_e5m2(self):
        return self.fp8_max == E5M2_MAX

    def _quant(self, x, scale):
        return (orc.quantize_e5m2 if self.is_e5m2() else orc.quantize_e4m3)(x, scale)

    def quant_act(self, x, is_recompute=False):
        """x: bf16 bit patterns.  Returns the quantized bytes."""
        if is_recompute:                                                   # src/trainer.cu:4736-4743
            return self._quant(x, self.scale_snapshot)
        if self.calib_commit_pending:                                      # src/trainer.cu:4747-4768
            self.calib_commit_pending = False
            spread = self.calib_max / self.calib_min if self.calib_min > 0 else np.float32(0)
            if self.fp8_max == E4M3_MAX and spread > self.spread_threshold:
                self.fp8_max = E5M2_MAX
                self.amax = self.calib_max
                self.delayed.cursor[0] = 0
                self.delayed.count[0] = 0
                s, d = orc.scale_from_amax(self.amax, self.fp8_max)
                self.delayed.scale[0], self.delayed.descale[0] = s, d
                self.delayed.update(self.amax, self.fp8_max)
        self.amax = np.float32(0)                                          # src/trainer.cu:4770
        if self.calib_remaining > 0 or not self.init:                      # src/trainer.cu:4771-4818
            self.amax = orc.amax_bf16(x)
            s, d = orc.scale_from_amax(self.amax, self.fp8_max)
            self.delayed.scale[0], self.delayed.descale[0] = s, d
            self.scale_snapshot, self.descale_snapshot = s, d
            q = self._quant(x, s)
            if self.calib_remaining > 0:
                self.calib_min, self.calib_max = orc.calib_minmax_update(self.amax, self.calib_min, self.calib_max)
            self.delayed.update(self.amax, self.fp8_max)
            self.init = True
            if self.calib_remaining > 0:
                self.calib_remaining -= 1
                if self.calib_remaining == 0:
                    self.calib_commit_pending = True
            return q
        self.scale_snapshot, self.descale_snapshot = self.scale, self.descale      # src/trainer.cu:4823-4826
        q, self.amax = orc.quantize_record(x, self.scale, self.amax, e5m2=self.is_e5m2())
        self.delayed.update(self.amax, self.fp8_max)                                # src/trainer.cu:4840-4850
        return q


def refresh_weight(w_bits, in_dim, out_dim, stored_out_major, amax=None):
    """One Fp8Slot of refresh_fp8_weights (src/trainer.cu:4694-4712).  Returns fwd8 [out,in], bwd8 [in,out], amax, scale, descale."""
    if amax is None:
        amax = orc.amax_bf16(w_bits)
    s, d = orc.scale_from_amax(amax, 448.0)
    if stored_out_major:
        w2 = w_bits.reshape(out_dim, in_dim)
        return orc.quantize_e4m3(w2, s), orc.quantize_transpose_e4m3(w2, s), amax, s, d
    w2 = w_bits.reshape(in_dim, out_dim)
    return orc.quantize_transpose_e4m3(w2, s), orc.quantize_e4m3(w2, s), amax, s, d
