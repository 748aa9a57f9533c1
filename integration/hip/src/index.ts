/**
 * @alpha/hip -- registers the MI355X backend under the name "hip", the way the Vulkan backend registers itself
 * (packages/helios/src/index.ts:29-30).  The CLI merges backend registries by name (apps/cli/src/resolve.ts:12-19):
 *
 *     import { hipRegistry } from "@alpha/hip";
 *     for (const name of hipRegistry.list()) backendRegistry.register(name, () => hipRegistry.get(name));
 *
 * after which `alpha train --backend=hip` runs the unchanged packages/train loop on libalpha_hip.so.  The class has no
 * `smokeTest` member: the trainer's smoke-test path is guarded for NVIDIA device names (packages/train/src/trainer.ts:623,
 * 757-841) and is skipped for a backend that does not offer one.
 */
export { HipBackend, type HipDeviceInfo } from "./backend.js";
export { lib as hipLibrary, check as hipCheck, LAYOUT as hipStructLayout } from "./ffi.js";
export type { Backend, TensorData, Dtype, Shape } from "@alpha/core";

import { Registry } from "@alpha/core";
import type { Backend } from "@alpha/core";
import { HipBackend } from "./backend.js";

export const hipRegistry = new Registry<Backend>("backend");
hipRegistry.register("hip", () => new HipBackend());
