"""MI355X-native rendering hot path of SplatAD behind the gsplat operator API."""
