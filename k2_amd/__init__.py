"""MI355X-native implementation of k2's RNN-T mutual-information path."""
