'use strict';
// DEBUG-mode kernel profiler, after tfjs-core/src/profiler.ts:24-74: times a kernel with
// backend.time(), downloads every output, checks it for NaN/Infinity and logs one line.
class Profiler {
  constructor(backendTimer, logger) {
    this.backendTimer = backendTimer;
    this.logger = logger || new Logger();
  }
  profileKernel(name, f) {
    let result;
    const holdResultWrapperFn = () => { result = f(); };
    const timer = this.backendTimer.time(holdResultWrapperFn);
    const results = Array.isArray(result) ? result : [result];
    results.forEach(r => {
      const vals = r.dataSync();
      checkComputationForErrors(vals, r.dtype, name);
      timer.then(timing => {
        let extraInfo = '';
        if (timing.getExtraProfileInfo != null) extraInfo = timing.getExtraProfileInfo();
        this.logger.logKernelProfile(name, r, vals, timing.kernelMs, extraInfo);
      });
    });
    return result;
  }
}

function checkComputationForErrors(vals, dtype, name) {
  if (dtype !== 'float32') return false;
  for (let i = 0; i < vals.length; i++) {
    const num = vals[i];
    if (isNaN(num) || !isFinite(num)) {
      console.warn(`Found ${num} in the result of '${name}'`);
      return true;
    }
  }
  return false;
}

class Logger {
  logKernelProfile(name, result, vals, timeMs, extraInfo) {
    const time = (typeof timeMs === 'number' ? timeMs.toFixed(3) : timeMs) + 'ms';
    console.log(`${name}\t${time}\t${result.rank}D ${JSON.stringify(result.shape)}\t${result.size}\t${extraInfo || ''}`);
  }
}

module.exports = {Profiler, Logger, checkComputationForErrors};
